"""Glue registry: maps a tensor class to the glue module that handles it,
importing that module on first use (reference: mobula/glue/backend.py)."""
import importlib
from itertools import chain

from .common import MobulaTensor

DTYPE_TO_GLUE = {}       # tensor class -> glue module
GLUE_NAME_TO_GLUE = {}   # 'torch' -> glue module
PKG_NAME_TO_GLUE_ARGS = {}  # top-level package name -> (glue name, [class paths])


def register_glue(glue_name, type_names):
    assert type_names, ValueError('type_names should be not empty')
    pkgs = {path.split('.')[0] for path in type_names}
    assert len(pkgs) == 1, TypeError(
        'The name of package should be consistent in `types_name`: {}'.format(type_names))
    PKG_NAME_TO_GLUE_ARGS[pkgs.pop()] = (glue_name, list(type_names))


register_glue('numpy', ['numpy.ndarray'])
register_glue('torch', ['torch.Tensor'])


def _resolve(path):
    parts = path.split('.')
    obj = importlib.import_module(parts[0])
    for attr in parts[1:]:
        obj = getattr(obj, attr, None)
        if obj is None:
            raise ImportError(path)
    return obj


def _activate(glue_name, type_names):
    try:
        glue = importlib.import_module('.{}_glue'.format(glue_name), __package__)
    except ImportError:
        return
    assert callable(getattr(glue.OpGen, '__call__', None)) and hasattr(glue.OpGen, 'register')
    if not hasattr(glue, 'Tensor'):
        found = [v for k, v in vars(glue).items()
                 if isinstance(v, type) and issubclass(v, MobulaTensor)
                 and k.lower() == glue_name + 'tensor']
        assert len(found) == 1, 'Only one MobulaTensor is allowed in each glue module'
        glue.Tensor = found[0]
    glue.gen_cache = {}
    for path in type_names:
        try:
            DTYPE_TO_GLUE[_resolve(path)] = glue
        except ImportError:
            pass
    GLUE_NAME_TO_GLUE[glue_name] = glue


def get_var_type_glue(vtype):
    """Glue module for a tensor class, or None."""
    glue = DTYPE_TO_GLUE.get(vtype)
    if glue is not None:
        return glue
    for klass in getattr(vtype, '__mro__', ()):  # subclasses (e.g. nn.Parameter)
        if klass in DTYPE_TO_GLUE:
            return DTYPE_TO_GLUE[klass]
    pkg = getattr(vtype, '__module__', '').split('.')[0]
    if pkg not in PKG_NAME_TO_GLUE_ARGS:
        return None
    if PKG_NAME_TO_GLUE_ARGS[pkg][0] not in GLUE_NAME_TO_GLUE:
        _activate(*PKG_NAME_TO_GLUE_ARGS[pkg])
    for klass in getattr(vtype, '__mro__', (vtype,)):
        if klass in DTYPE_TO_GLUE:
            return DTYPE_TO_GLUE[klass]
    return None


def get_var_glue(var):
    return get_var_type_glue(type(var))


def get_args_glue(*args, **kwargs):
    """The single glue module all tensor arguments belong to (None if no tensors)."""
    mods = [m for m in map(get_var_glue, chain(args, kwargs.values())) if m is not None]
    if not mods:
        return None
    assert all(m is mods[0] for m in mods), TypeError(
        'Support only 1 backend in a call, now: {}'.format(mods))
    return mods[0]


def op_gen(glue_mod, op, name):
    if name not in glue_mod.gen_cache:
        glue_mod.gen_cache[name] = glue_mod.OpGen(op=op, name=name)
    return glue_mod.gen_cache[name]


def get_glue_modules():
    return GLUE_NAME_TO_GLUE.values()
