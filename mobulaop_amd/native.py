"""Loading of the HIP launcher library and its per-call side channel.

The library (`csrc/libmobula_hip.so`, built by `mobulaop_amd.build`) exports the
operator entry points under the reference's naming scheme plus a few
`mobula_hip_*` control functions:

  mobula_hip_set_stream(stream, synchronous)   thread-local launch stream
  mobula_hip_set_arg_extents(numel[], n)       element counts of the next call's
                                               arguments (-1 for scalars)
  mobula_hip_last_error() / clear_error()      error text of the last failed call
  mobula_hip_set_option(name, value)           tuning / implementation switches

There is no CPU implementation behind this module: if the library is missing
(and cannot be built) every call raises.
"""
import ctypes
import os

from .config import config
from .dtype import CTYPENAME2CTYPE

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'csrc', 'libmobula_hip.so')

_lib = None


def ctype_by_name(name):
    return CTYPENAME2CTYPE[name]


def library():
    """The launcher CDLL; builds it first if it is absent and hipcc exists."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            from . import build as _build
            _build.build_library()
        try:
            lib = ctypes.CDLL(LIB_PATH)
        except OSError as exc:
            raise RuntimeError('cannot load the HIP launcher library {}: {} -- build it with '
                               '`python -m mobulaop_amd.build`'.format(LIB_PATH, exc))
        lib.mobula_hip_last_error.restype = ctypes.c_char_p
        lib.mobula_hip_set_stream.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.mobula_hip_set_arg_extents.argtypes = [ctypes.POINTER(ctypes.c_longlong), ctypes.c_int]
        lib.mobula_hip_set_option.argtypes = [ctypes.c_char_p, ctypes.c_longlong]
        lib.mobula_hip_set_option.restype = ctypes.c_int
        lib.mobula_hip_get_option.argtypes = [ctypes.c_char_p]
        lib.mobula_hip_get_option.restype = ctypes.c_longlong
        _lib = lib
        _push_config()
    return _lib


_IMPL_CODES = {'auto': 0, 'tiled': 1, 'naive': 2}


def _push_config():
    set_option('roialign_impl', _IMPL_CODES[config.ROIALIGN_IMPL])
    set_option('host_staging_device', config.HOST_STAGING_DEVICE)


def set_option(name, value):
    if library().mobula_hip_set_option(name.encode(), int(value)) != 0:
        raise KeyError('unknown launcher option {!r}'.format(name))


def get_option(name):
    return int(library().mobula_hip_get_option(name.encode()))


def symbol(name):
    """Exported function `name`, or None."""
    try:
        return getattr(library(), name)
    except AttributeError:
        return None


def exported_names():
    """Names of the operator entry points the library says it exports."""
    lib = library()
    lib.mobula_hip_exports.restype = ctypes.c_char_p
    return lib.mobula_hip_exports().decode().split()


def roialign_channels_last_supported(backward, elem_bytes, channels, height, width, pooled_size,
                                     sampling_ratio, num_rois):
    """True if the channels-last ROIAlign entry points take this shape."""
    fn = symbol('mobula_hip_roialign_nhwc_supported')
    if fn is None:
        return False
    fn.argtypes = [ctypes.c_int] * 8 + [ctypes.c_longlong]
    fn.restype = ctypes.c_int
    return bool(fn(int(bool(backward)), int(elem_bytes), int(channels), int(height), int(width),
                   int(pooled_size[0]), int(pooled_size[1]), int(sampling_ratio), int(num_rois)))


def device_can_read(address):
    """True if a kernel may dereference `address` (device, pinned or managed memory)."""
    fn = library().mobula_hip_device_can_read
    fn.argtypes = [ctypes.c_void_p]
    fn.restype = ctypes.c_int
    return bool(fn(ctypes.c_void_p(address)))


def workspace_bytes():
    """Size of the calling thread's scratch buffer on the current device."""
    fn = library().mobula_hip_workspace_bytes
    fn.restype = ctypes.c_longlong
    return int(fn())


def release_workspace():
    """Give the calling thread's scratch buffer back to the device; returns the
    bytes freed.  The next call allocates what it needs.  Refused (RuntimeError)
    while a recorded HIP graph uses the buffer: see unpin_workspace()."""
    lib = library()
    fn = lib.mobula_hip_release_workspace
    fn.restype = ctypes.c_longlong
    freed = int(fn())
    msg = lib.mobula_hip_last_error()
    if msg:
        text = msg.decode()
        lib.mobula_hip_clear_error()
        raise RuntimeError(text)
    return freed


def unpin_workspace():
    """Tell the library that no recorded HIP graph uses the calling thread's scratch
    buffer any more (recording a call pins it: it is then neither grown nor released)."""
    library().mobula_hip_unpin_workspace()


def begin_call(stream, extents):
    lib = library()
    if stream is None:
        lib.mobula_hip_set_stream(None, 1)
    else:
        lib.mobula_hip_set_stream(ctypes.c_void_p(stream), 0)
    arr = (ctypes.c_longlong * len(extents))(*extents)
    lib.mobula_hip_set_arg_extents(arr, len(extents))


def end_call(func_name):
    lib = library()
    msg = lib.mobula_hip_last_error()
    if msg:
        text = msg.decode()
        lib.mobula_hip_clear_error()
        raise RuntimeError('{}: {}'.format(func_name, text))
