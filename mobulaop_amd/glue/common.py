"""Pieces shared by the framework glues (reference: mobula/glue/common.py).

An operator class provides `forward(self, *inputs)`, `backward(self, *out_grads)`
and `infer_shape(self, in_shape)`.  The glue injects `in_data/out_data/in_grad/
out_grad`, `req`, `F` and the accessors `X Y dX dY x y dx dy` before calling it.
"""
import ctypes
import functools
import inspect
import warnings

import numpy as np

from ..dtype import c_half

CUSTOM_OP_LIST = {}
CSTRUCT_CONSTRUCTOR = {}  # structure name in operator sources -> (ctypes.Structure class, constructor)


def register_cstruct(name, cstruct, constructor=None):
    """Let operator sources loaded from now on take `name*` parameters: a call passes
    either what `constructor` accepts (default: the structure class itself) or a tuple
    of its positional arguments (reference: mobula/glue/common.py:197-202)."""
    if constructor is None:
        constructor = cstruct
    assert callable(constructor), 'constructor {} should be callable'.format(name)
    CSTRUCT_CONSTRUCTOR[name] = (cstruct, constructor)

OP_MODULE_GLOBALS = None  # set to mobula.op's namespace when that package is imported
backend = None            # set by glue/__init__.py


@functools.lru_cache(maxsize=None)
def _argspec_of_function(func):
    return inspect.getfullargspec(func)


def _argspec(func):
    """Signature of a method, looked up once per underlying function (the calls
    below sit on the per-invocation path of every operator)."""
    return _argspec_of_function(getattr(func, '__func__', func))


def get_varnames(func):
    """Positional parameter names of a method, without `self`."""
    return _argspec(func).args[1:]


def get_in_data(*args, **kwargs):
    """Split a call `Op(*args, **kwargs)` into tensor inputs (the parameters of
    `op.forward`) and constructor parameters (everything else).

    Returns (inputs, [ctor_args, ctor_kwargs])  (reference: common.py:68-105)."""
    op = kwargs.pop('op')
    spec = _argspec(op.forward)
    names = spec.args[1:]
    n_in = len(names)
    n_opt = len(spec.defaults) if spec.defaults else 0
    if len(args) >= n_in:
        return args[:n_in], [args[n_in:], kwargs]
    inputs = list(args)
    for name in names[:len(args)]:
        assert name not in kwargs, 'Variable %s given twice' % name
    for i in range(len(args), n_in - n_opt):  # required inputs must be present
        assert names[i] in kwargs, 'Variable %s not found' % names[i]
        inputs.append(kwargs.pop(names[i]))
    for i in range(max(len(args), n_in - n_opt), n_in):  # optional ones stop at the first gap
        if names[i] not in kwargs:
            break
        inputs.append(kwargs.pop(names[i]))
    return inputs, [[], kwargs]


def get_in_shape(in_data):
    return [d.shape for d in in_data]


def assign(_, dst, req, src):
    """Store `src` into `dst` according to the write request."""
    if req == 'null':
        return
    if req in ('write', 'inplace'):
        dst[:] = src
    elif req == 'add':
        dst[:] += src


class MobulaTensor:
    """Uniform view of a framework tensor for the function binding: raw
    pointer (plus a contiguous temporary when needed), element ctype, device."""
    F = None

    def __init__(self, tensor):
        self.tensor = tensor

    @property
    def data_ptr(self):
        raise NotImplementedError

    @property
    def ctype(self):
        raise NotImplementedError

    @property
    def dev_id(self):
        raise NotImplementedError

    @property
    def numel(self):
        raise NotImplementedError


class MobulaOperator:
    """Callable handle stored as `mobula.op.<Name>`.

    `Op(*tensors, **ctor_kwargs)` dispatches on the tensors' framework;
    `Op[np.ndarray](**ctor_kwargs)` returns a stateful op object of that glue."""

    def __init__(self, op, name, **attrs):
        self.op = op
        self.name = name
        self.attrs = attrs

    def __call__(self, *args, **kwargs):
        glue_mod = backend.get_args_glue(*args, **kwargs)
        assert glue_mod is not None, ValueError('No explict backend')
        merged = dict(kwargs)
        merged.update(self.attrs)
        return backend.op_gen(glue_mod, op=self.op, name=self.name)(*args, **merged)

    def __getitem__(self, input_type):
        glue_mod = backend.get_var_type_glue(input_type)
        assert glue_mod is not None, ValueError(
            'The backend of {} is not found'.format(input_type))

        def make(*args, **kwargs):
            merged = dict(kwargs)
            merged.update(self.attrs)
            merged['__input_type__'] = input_type
            return backend.op_gen(glue_mod, op=self.op, name=self.name)(*args, **merged)
        return make


def register(op_name=None, **attrs):
    """`@register`, `@register('Name')` or `@register(attr=value)` on an op class."""
    def bind(name, cls):
        name = name or cls.__name__
        handle = MobulaOperator(op=cls, name=name, **attrs)
        if name in CUSTOM_OP_LIST:
            warnings.warn('Duplicate operator name {}, please rename it'.format(name))
        CUSTOM_OP_LIST[name] = handle
        if OP_MODULE_GLOBALS is not None:
            OP_MODULE_GLOBALS[name] = handle
        return handle
    if op_name is not None and not isinstance(op_name, str):
        return bind(None, op_name)  # bare decorator: op_name is the class
    return functools.partial(bind, op_name)


INPUT_FUNCS = dict(
    X=property(lambda self: self.in_data),
    Y=property(lambda self: self.out_data),
    dX=property(lambda self: self.in_grad),
    dY=property(lambda self: self.out_grad),
    x=property(lambda self: self.in_data[0]),
    y=property(lambda self: self.out_data[0]),
    dx=property(lambda self: self.in_grad[0]),
    dy=property(lambda self: self.out_grad[0]),
)

_NP2CTYPE = {
    'int8': ctypes.c_int8, 'int16': ctypes.c_int16, 'int32': ctypes.c_int32,
    'int64': ctypes.c_int64, 'float32': ctypes.c_float, 'float64': ctypes.c_double,
    'float16': c_half,  # extension: fp16 storage
}


def NPDTYPE2CTYPE(dtype):
    ctype = _NP2CTYPE.get(np.dtype(dtype).name)
    assert ctype is not None, TypeError('Unknown Type: {}'.format(dtype))
    return ctype
