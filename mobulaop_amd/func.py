"""Function binding: `mobula.func.<name>(*args, **kwargs)` -> one foreign call
into the HIP launcher library (reference: mobula/func.py).

What is kept from the reference, because callers can observe it:
  * keyword arguments are appended in declaration order (func.py:190-194);
  * the first tensor bound to a template parameter fixes its C type, later
    ones must agree, template scalars take that type (func.py:247-306);
  * all tensors of one call live on one device (func.py:239-245);
  * non-contiguous tensors are passed as contiguous temporaries and mutable
    ones are copied back afterwards (func.py:79-92,162-163);
  * the exported symbol is `<func>_<md5(','.join(argument C names))[:8]>`
    and kernels receive the device id as an extra first argument, -1 for host
    memory (func.py:13-50,138-156).
What is new: the launcher is told, per call and per thread, which HIP stream to
use and how many elements each pointer argument holds (so that it can validate
shapes before launching), and HIP errors come back as RuntimeError instead of
terminating the process.
"""
import ctypes
import hashlib
import warnings

from . import glue
from . import native
from .config import config
from .dtype import CStruct, DType, TemplateType, UnknownCType

__all__ = ['MobulaFunc', 'CFuncDef', 'bind', 'get_func_idcode', 'get_idcode_hash']


def get_func_idcode(func_name, arg_types):
    return '{}:{}'.format(func_name, ','.join(t.cname for t in arg_types))


def get_idcode_hash(idcode):
    func_name, _, signature = idcode.partition(':')
    return '{}_{}'.format(func_name, hashlib.md5(signature.encode('utf-8')).hexdigest()[:8])


_DTYPES = {}


def _dtype(ctype, is_const):
    """The one DType instance for (ctype, constness): descriptors are immutable, and
    sharing them lets a call's resolved symbol be looked up by the identity of its
    argument types."""
    key = (ctype, is_const)
    found = _DTYPES.get(key)
    if found is None:
        found = _DTYPES[key] = DType(ctype, is_const=is_const)
    return found


class _TensorArg:
    __slots__ = ('var', 'ptype', 'view')

    def __init__(self, var, ptype, view):
        self.var = var
        self.ptype = ptype
        self.view = view  # glue Tensor wrapper


class _StructArg:
    """A registered structure, passed by address."""
    __slots__ = ('value',)

    def __init__(self, value):
        self.value = value


def _pointer_fields(value):
    """(field path, address) of every non-null pointer field of a ctypes structure,
    nested structures included."""
    for name, ftype in getattr(value, '_fields_', ()):
        field = getattr(value, name)
        if isinstance(field, ctypes.Structure):
            for sub, addr in _pointer_fields(field):
                yield name + '.' + sub, addr
        elif isinstance(field, ctypes._Pointer):
            addr = ctypes.cast(field, ctypes.c_void_p).value
            if addr:
                yield name, addr
        elif ftype is ctypes.c_void_p and field:
            yield name, int(field)


class CFuncDef:
    """Declaration of one exported function, as parsed from the op source."""
    KERNEL = 1
    FUNC = 2

    def __init__(self, func_name, func_kind, arg_names=None, arg_types=None, rtn_type=None,
                 template_list=None, loader=None, loader_kwargs=None, template_defaults=None):
        self.func_name = func_name
        self.func_kind = func_kind
        self.arg_names = arg_names or []
        self.arg_types = arg_types
        self.rtn_type = rtn_type
        self.template_list = template_list or []
        self.template_defaults = template_defaults or {}   # `typename B = T` -> {'B': 'T'}
        self.loader = loader
        self.loader_kwargs = loader_kwargs or {}
        self._resolved = {}

    def __call__(self, arg_datas, arg_types, dev_id, glue_mod=None, using_async=False):
        ctx = 'cpu' if dev_id is None else config.GPU_BACKEND
        # the symbol of an instantiation, remembered by the (shared) type descriptors
        key = (ctx,) + tuple(map(id, arg_types))
        cfunc = self._resolved.get(key)
        if cfunc is None:
            cfunc = self.loader(self, arg_types, ctx, **self.loader_kwargs)
            if all(_DTYPES.get((getattr(t, 'ctype', None), t.is_const)) is t or isinstance(t, CStruct)
                   for t in arg_types):
                self._resolved[key] = cfunc   # ids of shared descriptors never get reused

        keep_alive, copy_back, raw, extents = [], [], [], []
        for arg in arg_datas:
            if isinstance(arg, _TensorArg):
                ptr = arg.view.data_ptr
                if isinstance(ptr, (list, tuple)):
                    ptr, dense = ptr
                    keep_alive.append(dense)
                    if not arg.ptype.is_const:
                        copy_back.append((arg.var, dense))
                raw.append(ptr)
                extents.append(int(arg.view.numel))
            elif isinstance(arg, _StructArg):
                if self.func_kind == CFuncDef.KERNEL:
                    # the kernel reads the structure's copy on the GPU and follows its pointers there
                    for path, addr in _pointer_fields(arg.value):
                        if not native.device_can_read(addr):
                            raise TypeError(
                                '{}: field `{}` of the structure argument points to ordinary host memory, '
                                'which a kernel cannot read; build the structure from a GPU tensor'.format(
                                    self.func_name, path))
                keep_alive.append(arg.value)
                raw.append(ctypes.byref(arg.value))
                extents.append(1)
            else:
                raw.append(arg)
                extents.append(-1)

        if self.func_kind == CFuncDef.KERNEL:
            stream = None
            if dev_id is not None and glue_mod is not None and hasattr(glue_mod, 'current_stream'):
                stream = glue_mod.current_stream(dev_id)
            native.begin_call(stream=stream, extents=extents)
            out = cfunc(ctypes.c_int(-1 if dev_id is None else dev_id), *raw)
            native.end_call(self.func_name)
        elif self.func_kind == CFuncDef.FUNC:
            # a host function; if it launches kernels itself they go to the tensors'
            # stream, and what it reports as fatal is raised here
            stream = None
            if dev_id is not None and glue_mod is not None and hasattr(glue_mod, 'current_stream'):
                stream = glue_mod.current_stream(dev_id)
            native.begin_call(stream=stream, extents=extents)
            out = cfunc(*raw)
            native.end_call(self.func_name)
        else:
            raise TypeError('Unsupported func kind: {}'.format(self.func_kind))
        for target, dense in copy_back:
            target[:] = dense
        return out


class MobulaFunc:
    """Python callable for one exported function."""

    def __init__(self, name, func):
        self.name = name
        self.func = func

    def __call__(self, *args, **kwargs):
        decl = self.func
        args = list(args)
        for name in decl.arg_names[len(args):]:
            args.append(kwargs[name])

        if len(args) != len(decl.arg_types):
            raise TypeError('Unmatched parameters list of the function `{}`: expected {} arguments, '
                            'got {}'.format(self.name, len(decl.arg_types), len(args)))
        arg_datas, arg_types = [], []
        template_map = {}
        dev_id = None
        placement = None
        glue_mod = self._common_glue(args)
        try:
            for var, ptype in zip(args, decl.arg_types):
                if isinstance(ptype, CStruct):
                    if isinstance(var, ptype.cstruct):
                        value = var
                    else:
                        try:
                            value = ptype.constructor(var)
                        except TypeError:
                            value = ptype.constructor(*var)
                    arg_datas.append(_StructArg(value))
                    arg_types.append(ptype)
                    continue
                if ptype.is_pointer and not (isinstance(ptype, DType) and
                                             ptype.ctype is ctypes.c_void_p):
                    data, var_dev, ctype = self._tensor_info(var, ptype, template_map)
                    # host memory counts as a device of its own: a host pointer
                    # must never reach a kernel that expects device memory
                    where = 'host' if var_dev is None else var_dev
                    placement = where if placement is None else placement
                    assert where == placement, ValueError(
                        "Don't use multiple devices in a call :-(")
                    dev_id = var_dev
                else:
                    data, ctype = self._scalar_info(var, ptype)
                arg_datas.append(data)
                if isinstance(ctype, UnknownCType):
                    ctype.is_const = ptype.is_const
                    arg_types.append(ctype)
                else:
                    arg_types.append(_dtype(ctype, ptype.is_const))
            for i, t in enumerate(arg_types):  # template scalars: type known only now
                if isinstance(t, UnknownCType):
                    assert t.tname in template_map, Exception(
                        'Unknown template name: {}'.format(t.tname))
                    scalar_ctype = template_map[t.tname]._type_
                    arg_types[i] = _dtype(scalar_ctype, t.is_const)
                    arg_datas[i] = scalar_ctype(arg_datas[i])
        except TypeError:
            raise TypeError('Unmatched parameters list of the function `{}`:\n\t{}\n\t\tvs\n\t{}'
                            .format(self.name, decl.arg_types, [type(a) for a in args]))
        return decl(arg_datas=arg_datas, arg_types=arg_types, dev_id=dev_id, glue_mod=glue_mod)

    @staticmethod
    def _tensor_info(var, ptype, template_map):
        glue_mod = glue.backend.get_var_glue(var)
        if glue_mod is None:
            raise TypeError()
        view = glue_mod.Tensor(var)
        ctype = ctypes.POINTER(view.ctype)
        if isinstance(ptype, DType):
            expected = ptype.ctype
        else:
            expected = template_map.setdefault(ptype.tname, ctype)
        assert ctype == expected, TypeError(
            'Expected Type {} instead of {}'.format(expected, ctype))
        return _TensorArg(var, ptype, view), view.dev_id, ctype

    @staticmethod
    def _scalar_info(var, ptype):
        if isinstance(ptype, TemplateType):
            if hasattr(var, '_type_'):  # already a ctypes scalar: its type wins
                return var, type(var)
            return var, UnknownCType(ptype.tname)
        if isinstance(var, ctypes.c_void_p):
            return var, ptype.ctype
        return ptype.ctype(var), ptype.ctype

    @staticmethod
    def _common_glue(values):
        mods = [m for m in map(glue.backend.get_var_glue, values) if m is not None]
        if mods and all(m is mods[0] for m in mods):
            return mods[0]
        return None

    def build(self, ctx, template_types=None):
        """Resolve (and thereby check the presence of) one instantiation, e.g.
        `mobula.func.roi_align_forward.build('hip', ['float', 'float'])`."""
        decl = self.func
        pending = list(template_types) if isinstance(template_types, (list, tuple)) else None
        by_name = dict(template_types) if isinstance(template_types, dict) else {}
        arg_types = []
        for t in decl.arg_types:
            if isinstance(t, TemplateType):
                if t.tname not in by_name:
                    if pending:
                        by_name[t.tname] = pending.pop(0)
                    else:  # a default names a type, or a parameter given before it
                        default = decl.template_defaults.get(t.tname)
                        assert default is not None, Exception(
                            'missing template type for {}'.format(t.tname))
                        by_name[t.tname] = by_name.get(default, default)
                arg_types.append(t(getattr(ctypes, 'c_' + by_name[t.tname], None) or
                                   native.ctype_by_name(by_name[t.tname])))
            else:
                arg_types.append(t)
        assert not pending, Exception('redundant type')
        decl.loader(decl, arg_types, ctx, **decl.loader_kwargs)


_bound = {}


def bind(functions):
    """Publish `name -> CFuncDef` as `mobula.func.<name>`."""
    for name, decl in functions.items():
        if name in _bound:
            warnings.warn('Duplicated function name {}'.format(name))
        fn = MobulaFunc(name, decl)
        globals()[name] = fn
        _bound[name] = fn
