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


def _store(dst, src):
    dst[:] = src


def _accumulate(dst, src):
    dst[:] += src


_WRITERS = {'null': None, 'write': _store, 'inplace': _store, 'add': _accumulate}


def assign(_, dst, req, src):
    """`dst` receives `src` the way the write request says (bound as a method of
    the generated operator classes, hence the unused first parameter)."""
    writer = _WRITERS.get(req)
    if writer is not None:
        writer(dst, src)


def _required(name):
    def missing(self):
        raise NotImplementedError('{}.{}'.format(type(self).__name__, name))
    return property(missing)


class MobulaTensor:
    """What the function binding needs to know about a framework tensor; each glue
    derives one class from this and fills in the properties:

    data_ptr  raw address, or (address, contiguous temporary) for a strided tensor
    ctype     ctypes type of one element
    dev_id    None for host memory, else the device index
    numel     number of elements"""
    F = None   # the framework module (`numpy`, `torch`)
    data_ptr, ctype, dev_id, numel = (_required(n) for n in ('data_ptr', 'ctype', 'dev_id', 'numel'))

    def __init__(self, tensor):
        self.tensor = tensor


class MobulaOperator:
    """The handle stored as `mobula.op.<Name>`.

    `Op(*tensors, **params)` runs the operator in the framework of its tensors;
    `Op[tensor_type](**params)` makes an operator object of that framework without
    running it (the NumPy glue's objects have `.forward` / `.backward`)."""

    def __init__(self, op, name, **attrs):
        self.op, self.name, self.attrs = op, name, attrs

    def _generate(self, glue_mod, args, kwargs, **extra):
        return backend.op_gen(glue_mod, op=self.op, name=self.name)(
            *args, **dict(kwargs, **self.attrs, **extra))

    def __call__(self, *args, **kwargs):
        glue_mod = backend.get_args_glue(*args, **kwargs)
        assert glue_mod is not None, ValueError('No explict backend')
        return self._generate(glue_mod, args, kwargs)

    def __getitem__(self, input_type):
        glue_mod = backend.get_var_type_glue(input_type)
        assert glue_mod is not None, ValueError('The backend of {} is not found'.format(input_type))
        return lambda *args, **kwargs: self._generate(glue_mod, args, kwargs, __input_type__=input_type)


def _publish(cls, name, attrs):
    name = name or cls.__name__
    if name in CUSTOM_OP_LIST:
        warnings.warn('Duplicate operator name {}, please rename it'.format(name))
    handle = CUSTOM_OP_LIST[name] = MobulaOperator(op=cls, name=name, **attrs)
    if OP_MODULE_GLOBALS is not None:
        OP_MODULE_GLOBALS[name] = handle
    return handle


def register(op_name=None, **attrs):
    """Class decorator of operator modules: bare (`@register`), with a name
    (`@register('Name')`) or with attributes merged into every call
    (`@register(attr=value)`)."""
    if isinstance(op_name, type):          # bare: the argument is the class itself
        return _publish(op_name, None, attrs)
    return lambda cls: _publish(cls, op_name, attrs)


# Accessors the glues add to operator classes: X/Y/dX/dY are the lists of inputs,
# outputs and their gradients, the lower-case names their first elements.
_SLOTS = dict(X='in_data', Y='out_data', dX='in_grad', dY='out_grad')
INPUT_FUNCS = {}
for _short, _slot in _SLOTS.items():
    INPUT_FUNCS[_short] = property(lambda self, _slot=_slot: getattr(self, _slot))
    INPUT_FUNCS[_short.lower()] = property(lambda self, _slot=_slot: getattr(self, _slot)[0])

_NP2CTYPE = {
    'int8': ctypes.c_int8, 'int16': ctypes.c_int16, 'int32': ctypes.c_int32,
    'int64': ctypes.c_int64, 'float32': ctypes.c_float, 'float64': ctypes.c_double,
    'float16': c_half,  # extension: fp16 storage
}


def NPDTYPE2CTYPE(dtype):
    ctype = _NP2CTYPE.get(np.dtype(dtype).name)
    assert ctype is not None, TypeError('Unknown Type: {}'.format(dtype))
    return ctype
