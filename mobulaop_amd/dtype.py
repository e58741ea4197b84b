"""C type descriptors used to marshal arguments and to name exported symbols
(reference: mobula/internal/dtype.py:1-104).

The canonical C name of every argument type (`const float*`, `const int`, ...)
feeds the md5 that names the exported symbol, so it must agree with the
reference character for character for the types the reference knows.
"""
import ctypes


class c_half(ctypes.c_uint16):
    """IEEE binary16 storage.  Not in the reference (ctypes has no half type);
    added for the fp16-storage forward path.  Canonical C name: `half`."""


_LONG_SIGNED = (ctypes.c_long, ctypes.c_longlong)
_LONG_UNSIGNED = (ctypes.c_ulong, ctypes.c_ulonglong)

CTYPENAME2CTYPE = {
    'bool': ctypes.c_bool, 'char': ctypes.c_char, 'char*': ctypes.c_char_p,
    'double': ctypes.c_double, 'float': ctypes.c_float, 'half': c_half,
    'int': ctypes.c_int, 'int8_t': ctypes.c_int8, 'int16_t': ctypes.c_int16,
    'int32_t': ctypes.c_int32, 'int64_t': ctypes.c_int64, 'void*': ctypes.c_void_p,
    'void': None, None: None,
}


def ctype_basename(ctype):
    """`c_float` -> `float`, `c_long` -> `int64_t` (sized names for long types)."""
    if ctype in _LONG_SIGNED:
        return 'int{}_t'.format(8 * ctypes.sizeof(ctype))
    if ctype in _LONG_UNSIGNED:
        return 'uint{}_t'.format(8 * ctypes.sizeof(ctype))
    name = ctype.__name__
    return name[2:] if name.startswith('c_') else name


class DType:
    """A concrete C argument type: scalar or one-level pointer, const or not."""

    def __init__(self, ctype, is_const=False):
        self.ctype = ctype
        self.is_const = is_const
        self.is_pointer = ctype.__name__.startswith('LP_')
        base = ctype._type_ if self.is_pointer else ctype
        name = ctype_basename(base)
        if is_const:
            name = 'const ' + name
        self.cname = name + ('*' if self.is_pointer else '')

    def __repr__(self):
        return self.cname

    def __call__(self, value):
        return self.ctype(value)


class CStruct:
    """A pointer to a user structure registered with `mobula.glue.register_cstruct`
    (reference: mobula/internal/dtype.py:71-80).  The argument a caller passes is
    turned into the ctypes structure by `constructor`."""

    def __init__(self, name, is_const, cstruct, constructor):
        self.name = name
        self.cname = name + '*'     # constness is not part of the name, as in the reference
        self.cstruct = cstruct
        self.constructor = constructor
        self.is_pointer = True
        self.is_const = is_const

    def __repr__(self):
        return self.cname

    def __call__(self, *args, **kwargs):
        return self.constructor(*args, **kwargs)


class TemplateType:
    """An argument whose type is a template parameter (`T`, `const T*`, ...)."""

    def __init__(self, tname, is_pointer, is_const):
        self.tname = tname
        self.is_pointer = is_pointer
        self.is_const = is_const

    def __repr__(self):
        return '<typename {}{}{}>'.format('const ' if self.is_const else '', self.tname,
                                          '*' if self.is_pointer else '')

    def __call__(self, ctype):
        return DType(ctypes.POINTER(ctype) if self.is_pointer else ctype, self.is_const)


class UnknownCType:
    """Placeholder for a template scalar whose type is fixed by a later tensor."""

    def __init__(self, tname):
        self.tname = tname
        self.is_const = False
