"""`mobula.op.load(name, path='')`: publish an operator module.

An operator module is a directory `<Name>/` holding `<Name>.hip` (or `.cpp`)
with the `MOBULA_KERNEL` / `MOBULA_FUNC` launcher declarations and, optionally,
`<Name>.py` with the operator class.  Loading scans the source for the
declarations and binds one `mobula.func.<name>` per declaration, then executes
the Python file (reference: mobula/op/loader.py:538-659 for the scan and load,
:366-382 for symbol lookup).

The bundled operators (`.hip`: hand-written launchers) are compiled ahead of
time into the launcher library; resolving an instantiation of theirs that the
library does not export raises NameError with the list of what it does export.
A `.cpp` source in MobulaOP's kernel dialect (MOBULA_KERNEL + parfor) is
compiled on first use, one instantiation at a time (op/jit.py).
"""
import ctypes
import importlib.util
import os
import re

from ..dtype import DType, CStruct, TemplateType, CTYPENAME2CTYPE
from ..glue.common import CSTRUCT_CONSTRUCTOR
from ..func import CFuncDef, bind, get_func_idcode, get_idcode_hash
from .. import native

_TEMPLATE_RE = re.compile(r'^\s*template\s*<(.*?)>')
_HEAD_RE = re.compile(r'^\s*MOBULA_(KERNEL|FUNC)\b')
_DECL_RE = re.compile(r'^\s*MOBULA_(?:KERNEL|FUNC)\s+(.*?)\((.*)\)', re.S)

OPZOO_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), '..', 'opzoo')
_SOURCE_SUFFIXES = ('.hip', '.cpp')

# (ctx, idcode) -> ctypes function
_RESOLVED = {}


def _template_names(line):
    """`template <typename T, typename B = T>` -> (['T', 'B'], {'B': 'T'}); None if the
    line opens no template."""
    m = _TEMPLATE_RE.search(line)
    if m is None:
        return None
    names, defaults = [], {}
    for piece in m.group(1).split(','):
        piece, _, default = piece.partition('=')
        words = piece.split()
        if len(words) == 2 and words[0] in ('typename', 'class'):
            names.append(words[1])
            if default.strip():
                defaults[words[1]] = default.strip()
    return names, defaults


def parse_parameter_decl(decl):
    """`const T* bottom_data` -> (type descriptor, 'bottom_data')."""
    stars = decl.count('*')
    assert stars <= 1, Exception(
        'Only support pass-by-value or pass-by-1-level-pointer, Error declaration: ' + decl)
    words = decl.replace('*', ' ').split()
    is_const = words[0] == 'const'
    if is_const:
        words = words[1:]
    assert len(words) == 2, Exception('cannot parse parameter declaration: ' + decl)
    type_name, var_name = words
    is_pointer = stars == 1
    if type_name == 'void':
        assert is_pointer
        return DType(ctypes.c_void_p, is_const=is_const), var_name
    ctype = CTYPENAME2CTYPE.get(type_name) or getattr(ctypes, 'c_' + type_name, None)
    if ctype is not None:
        return DType(ctypes.POINTER(ctype) if is_pointer else ctype, is_const=is_const), var_name
    if type_name in CSTRUCT_CONSTRUCTOR:
        assert is_pointer, Exception('a registered structure is passed by pointer: ' + decl)
        cstruct, constructor = CSTRUCT_CONSTRUCTOR[type_name]
        return CStruct(type_name, is_const=is_const, cstruct=cstruct, constructor=constructor), var_name
    return TemplateType(tname=type_name, is_pointer=is_pointer, is_const=is_const), var_name


def parse_declaration(text):
    """`MOBULA_KERNEL foo_kernel(const int n, const T* a)` -> (rtn, name, [(type, name)...])."""
    m = _DECL_RE.search(text)
    assert m is not None, Exception('cannot parse declaration: ' + text)
    head = m.group(1).split()
    # the parameter list ends at the parenthesis that closes the first one (a body
    # on the same line may hold more)
    inner, depth = m.group(2), 1
    for i, ch in enumerate(inner):
        depth += {'(': 1, ')': -1}.get(ch, 0)
        if depth == 0:
            inner = inner[:i]
            break
    params = [p for p in (q.strip() for q in inner.split(',')) if p]
    rtn_type = head[-2] if len(head) >= 2 else None
    return rtn_type, head[-1], [parse_parameter_decl(p) for p in params]


class SourceInfo:
    def __init__(self, fname):
        self.cpp_fname = fname
        self.function_args = {}


class OpLoader:
    """Resolves one instantiation of a declared function to its exported symbol."""

    def __init__(self, cfunc, arg_types, ctx, cpp_info):
        idcode = get_func_idcode(cfunc.func_name, arg_types)
        key = (ctx, idcode)
        if key not in _RESOLVED:
            sym_name = get_idcode_hash(idcode)
            fn = native.symbol(sym_name)
            source = cpp_info.cpp_fname if cpp_info is not None else ''
            if fn is None and source.endswith('.cpp'):
                # an operator source in the kernel dialect: compiled on first use
                from . import jit
                fn = jit.resolve(cfunc, arg_types, source, sym_name)
            if fn is None:
                raise NameError('No function `{}` (symbol {}) in {}, current functions: {}'.format(
                    idcode, sym_name, native.LIB_PATH, native.exported_names()))
            rtn = cfunc.rtn_type
            if rtn in cfunc.template_list:   # the return type is a template parameter
                bound = [c.ctype for d, c in zip(cfunc.arg_types, arg_types)
                         if isinstance(d, TemplateType) and d.tname == rtn]
                assert bound, Exception('cannot tell the return type {} of {}'.format(rtn, cfunc.func_name))
                fn.restype = bound[0]._type_ if bound[0].__name__.startswith('LP_') else bound[0]
            else:
                fn.restype = CTYPENAME2CTYPE.get(rtn, None)
            _RESOLVED[key] = fn
        self.func = _RESOLVED[key]
        self.cpp_info = cpp_info
        self.idcode_hash = get_idcode_hash(idcode)

    def __call__(self, *args, **kwargs):
        return self.func(*args, **kwargs)


def _scan_source(fname):
    info = SourceInfo(fname)
    templates, defaults, pending, depth, kind = [], {}, None, 0, None
    with open(fname) as fin:
        for line in fin:
            if pending is None:
                names = _template_names(line)
                if names is not None:
                    templates, defaults = names
                m = _HEAD_RE.search(line)
                if m is None:
                    continue
                kind = CFuncDef.KERNEL if m.group(1) == 'KERNEL' else CFuncDef.FUNC
                pending, depth = '', 0
            depth += line.count('(') - line.count(')')
            pending += line.rstrip('\r\n') + ' '
            if depth != 0:
                continue
            rtn_type, cname, params = parse_declaration(pending)
            pending = None
            used = {t.tname for t, _ in params if isinstance(t, TemplateType)}
            assert len(set(templates)) == len(templates), Exception(
                'Duplicated template name in {}'.format(', '.join(templates)))
            for tname in used:
                assert tname in templates, Exception(
                    "template name '{}' is not defined".format(tname))
            if kind == CFuncDef.KERNEL:
                assert cname.endswith('_kernel'), Exception(
                    'the postfix of a MOBULA_KERNEL name must be `_kernel`, '
                    'e.g. addition_forward_kernel')
                func_name = cname[:-len('_kernel')]
            else:
                func_name = cname
            info.function_args[func_name] = dict(
                func_name=func_name, func_kind=kind,
                arg_names=[n for _, n in params], arg_types=[t for t, _ in params],
                rtn_type=rtn_type, template_list=list(templates) if used else [],
                template_defaults={k: v for k, v in defaults.items() if k in used},
                loader=OpLoader, loader_kwargs=dict(cpp_info=info))
            templates, defaults = [], {}
    assert pending is None, Exception('unbalanced parentheses in a declaration of ' + fname)
    return {name: CFuncDef(**kw) for name, kw in info.function_args.items()}


def load_module(name, pathname):
    spec = importlib.util.spec_from_file_location(name, pathname)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def load(module_name, path=''):
    """Load operator module `module_name` from `path` (default: the bundled opzoo,
    then the current directory)."""
    op_name = os.path.basename(module_name)
    if not path and os.path.exists(os.path.join(OPZOO_PATH, op_name)):
        path = OPZOO_PATH
    path = os.path.join(path, module_name)

    found = False
    for suffix in _SOURCE_SUFFIXES:
        src = os.path.join(path, op_name + suffix)
        if os.path.exists(src):
            found = True
            bind(_scan_source(src))
            break
    py_fname = os.path.join(path, op_name + '.py')
    if not os.path.exists(py_fname):
        py_fname = os.path.join(path, '__init__.py')
    if os.path.exists(py_fname):
        found = True
        load_module(op_name, py_fname)
    assert found, IOError('{0}.hip or {0}.cpp or {0}.py or __init__.py not found in the path {1}'
                          .format(op_name, path))
