"""Descriptors of C argument types.

Every parameter of an exported function is described by one of four kinds of
object, all answering `is_pointer`, `is_const` and (except the last two) `cname`:

* `DType`         a concrete scalar or one-level pointer (`const float*`, `int`)
* `CStruct`       a pointer to a registered user structure (`Span*`)
* `TemplateType`  a parameter whose type is a template parameter of the function
* `UnknownCType`  a template scalar in a call, until a tensor fixes its type

`cname` is the canonical spelling that is hashed into the exported symbol's name,
so for the types the reference knows it must agree with the reference character
for character (mobula/internal/dtype.py:23-62, mobula/func.py:13-50).
"""
import ctypes


class c_half(ctypes.c_uint16):
    """IEEE binary16 storage.  Not in the reference (ctypes has no half type);
    added for the fp16-storage paths.  Canonical C name: `half`."""


class c_bfloat16(ctypes.c_uint16):
    """bfloat16 storage (the upper half of a binary32), likewise an addition.
    Canonical C name: `bfloat16`."""


def _sized_name(ctype):
    """C `long` types are named by their width (`int64_t`), since their ctypes
    names differ between platforms."""
    signed = ctype in (ctypes.c_long, ctypes.c_longlong)
    if signed or ctype in (ctypes.c_ulong, ctypes.c_ulonglong):
        return '{}int{}_t'.format('' if signed else 'u', 8 * ctypes.sizeof(ctype))
    return None


def ctype_basename(ctype):
    """`c_float` -> `float`, `c_long` -> `int64_t`, `c_half` -> `half`."""
    return _sized_name(ctype) or ctype.__name__[2 if ctype.__name__.startswith('c_') else 0:]


CTYPENAME2CTYPE = dict(
    {name: getattr(ctypes, 'c_' + name) for name in
     ('bool', 'char', 'double', 'float', 'int', 'int8', 'int16', 'int32', 'int64')},
    half=c_half, bfloat16=c_bfloat16, void=None)
CTYPENAME2CTYPE.update({'char*': ctypes.c_char_p, 'void*': ctypes.c_void_p, None: None})
for _bits in (8, 16, 32, 64):   # the <cstdint> spellings
    CTYPENAME2CTYPE['int{}_t'.format(_bits)] = CTYPENAME2CTYPE.pop('int{}'.format(_bits))


class DType:
    __slots__ = ('ctype', 'is_const', 'is_pointer', 'cname')

    def __init__(self, ctype, is_const=False):
        pointee = getattr(ctype, '_type_', None) if ctype.__name__.startswith('LP_') else None
        self.ctype = ctype
        self.is_const = is_const
        self.is_pointer = pointee is not None
        self.cname = '{}{}{}'.format('const ' if is_const else '', ctype_basename(pointee or ctype),
                                     '*' if self.is_pointer else '')

    def __call__(self, value):
        return self.ctype(value)

    def __repr__(self):
        return self.cname


class CStruct:
    """Pointer to a structure registered with `mobula.glue.register_cstruct`
    (reference: mobula/internal/dtype.py:71-80): what a caller passes is turned into
    the ctypes structure by `constructor`.  Constness is not part of the name."""
    is_pointer = True

    def __init__(self, name, is_const, cstruct, constructor):
        self.name, self.cname = name, name + '*'
        self.cstruct, self.constructor = cstruct, constructor
        self.is_const = is_const

    def __call__(self, *args, **kwargs):
        return self.constructor(*args, **kwargs)

    def __repr__(self):
        return self.cname


class TemplateType:
    def __init__(self, tname, is_pointer, is_const):
        self.tname, self.is_pointer, self.is_const = tname, is_pointer, is_const

    def __call__(self, ctype):
        """The concrete descriptor once the parameter is bound to `ctype`."""
        return DType(ctypes.POINTER(ctype) if self.is_pointer else ctype, self.is_const)

    def __repr__(self):
        return '<typename {}{}{}>'.format('const ' if self.is_const else '', self.tname,
                                          '*' if self.is_pointer else '')


class UnknownCType:
    is_pointer = False

    def __init__(self, tname):
        self.tname = tname
        self.is_const = False
