"""Compile-on-load for operator sources written in MobulaOP's kernel dialect.

`mobula.op.load(name, path)` binds every `MOBULA_KERNEL` / `MOBULA_FUNC` of
`<path>/<name>/<name>.cpp`.  The launcher library knows nothing of such a
source, so the first call of a function with given argument types generates a
wrapper translation unit (the source itself plus one `extern "C"` entry point
named by the reference's scheme), compiles it with hipcc for gfx950 against
`inc/mobula_op.h`, and loads the result (reference: mobula/op/loader.py:405-526
with op/templates/kernel_code.cpp, func_code.cpp; there the whole operator is
rebuilt whenever a new instantiation appears, here every instantiation is a
shared object of its own, kept in `<operator directory>/build/`).
"""
import ctypes
import hashlib
import os
import re
import shutil
import stat
import subprocess

from ..config import config
from ..dtype import CStruct, DType, TemplateType
from ..func import CFuncDef
from .. import native

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC_PATH = os.path.join(_PKG, 'inc')
CSRC_PATH = os.path.join(_PKG, 'csrc')

# C spelling of the element types the binding knows (`half` and `bfloat16` are storage only)
_C_SPELLING = {'half': '__half', 'bfloat16': '__bf16'}

_loaded = {}


def _base_name(dtype):
    """`const float*` -> `float`."""
    name = dtype.cname
    if name.startswith('const '):
        name = name[len('const '):]
    return name.rstrip('*')


def _c_type(dtype):
    if isinstance(dtype, CStruct):
        return dtype.name + '*'   # converts to the kernel's `const Name*` where it asks for that
    base = _base_name(dtype)
    text = _C_SPELLING.get(base, base)
    if dtype.is_const:
        text = 'const ' + text
    return text + ('*' if dtype.is_pointer else '')


def _template_arguments(cfunc, arg_types):
    """Concrete type of every template parameter, in declaration order."""
    bound = {}
    for declared, concrete in zip(cfunc.arg_types, arg_types):
        if isinstance(declared, TemplateType):
            spelled = _C_SPELLING.get(_base_name(concrete), _base_name(concrete))
            assert bound.setdefault(declared.tname, spelled) == spelled, TypeError(
                'template parameter {} bound to two types'.format(declared.tname))
    return [bound[name] for name in cfunc.template_list]


_TOGETHER_RE = re.compile(r'\b(Reduce|__syncthreads|get_num_threads|get_thread_num)\b')


def kernel_body(text, kernel_name):
    """The text between the braces of `MOBULA_KERNEL <kernel_name>(...) {...}`, or ''."""
    m = re.search(r'MOBULA_KERNEL\s+' + re.escape(kernel_name) + r'\s*\(', text)
    if m is None:
        return ''
    i, depth = m.end(), 1
    while i < len(text) and depth:          # the parameter list
        depth += {'(': 1, ')': -1}.get(text[i], 0)
        i += 1
    start = text.find('{', i)
    if start < 0:
        return ''
    i, depth = start + 1, 1
    while i < len(text) and depth:
        depth += {'{': 1, '}': -1}.get(text[i], 0)
        i += 1
    return text[start + 1:i - 1]


def synchronises_its_threads(source, kernel_name):
    """True if the kernel must run as one workgroup: its body reduces over the
    launch, uses a barrier, or deals out work by thread number itself."""
    with open(source) as fin:
        text = re.sub(r'//[^\n]*|/\*.*?\*/', ' ', fin.read(), flags=re.S)
    return _TOGETHER_RE.search(kernel_body(text, kernel_name)) is not None


def wrapper_source(cfunc, arg_types, source, symbol, include=None):
    """The translation unit for one instantiation; `include` is how it names the
    operator source (default: its absolute path)."""
    names = cfunc.arg_names
    params = ', '.join('{} {}'.format(_c_type(t), n) for t, n in zip(arg_types, names))
    targs = _template_arguments(cfunc, arg_types)
    inst = '<{}>'.format(', '.join(targs)) if targs else ''
    lines = ['// generated: {} of {}'.format(symbol, os.path.basename(source)),
             '#include "mobula_op.h"', '#include "mobula_jit.h"', 'using namespace mobula;',
             '#include "{}"'.format(include or os.path.abspath(source)), '', 'extern "C" {']
    if cfunc.func_kind == CFuncDef.KERNEL:
        assert arg_types and not arg_types[0].is_pointer, TypeError(
            'the first parameter of a MOBULA_KERNEL is its iteration count')
        lines.append('void {}(const int device_id{}) {{'.format(symbol, ', ' + params if params else ''))
        lines.append('  mobula_jit::KernelCall call("{}", device_id);'.format(cfunc.func_name))
        passed = []
        for i, (t, n) in enumerate(zip(arg_types, names)):
            if isinstance(t, CStruct):
                lines.append('  {} {}_mapped = call.struct_arg({});'.format(_c_type(t), n, n))
                passed.append(n + '_mapped')
            elif t.is_pointer and _base_name(t) != 'void':
                lines.append('  {} {}_mapped = call.arg({}, {}, {});'.format(
                    _c_type(t), n, n, i, 'false' if t.is_const else 'true'))
                passed.append(n + '_mapped')
            else:
                passed.append(n)
        how = 'launch_together' if synchronises_its_threads(source, cfunc.func_name + '_kernel') else 'launch'
        lines.append('  call.{}({}, {}_kernel{}, {});'.format(how, names[0], cfunc.func_name, inst,
                                                             ', '.join(passed)))
        lines.append('}')
    else:
        # a host function: a failed CHECK / LOG(FATAL) becomes the call's error
        rtn = cfunc.rtn_type or 'void'
        if rtn in cfunc.template_list:   # `template <typename T> MOBULA_FUNC T f(...)`
            rtn = targs[cfunc.template_list.index(rtn)]
        lines.append('{} {}({}) {{'.format(rtn, symbol, params))
        lines.append('  try {')
        lines.append('    {}{}{}({});'.format('' if rtn == 'void' else 'return ', cfunc.func_name, inst,
                                              ', '.join(names)))
        lines.append('  } catch (const mobula::FatalError& e) {')
        lines.append('    mobula_hip::set_error("%s", e.what());')
        lines.append('  }')
        if rtn != 'void':
            lines.append('  return {}();'.format(rtn))
        lines.append('}')
    lines.append('}  // extern "C"')
    return '\n'.join(lines) + '\n'


def _build_dir(source):
    here = os.path.dirname(os.path.abspath(source))
    if not config.BUILD_IN_LOCAL_PATH:
        # reference: mobula/building/build_path.py:7-20
        tag = hashlib.md5(os.path.dirname(here).encode()).hexdigest()[:8]
        path = os.path.normpath(os.path.join(config.BUILD_PATH, 'build',
                                             '{}_{}'.format(os.path.basename(here), tag)))
        os.makedirs(path, exist_ok=True)
        return path
    path = os.path.join(here, 'build')
    # beside the source only if that directory is marked writable for its owner:
    # os.access() says yes to root for a tree that was deliberately made read-only
    try:
        if os.stat(here).st_mode & stat.S_IWUSR and os.access(here, os.W_OK):
            os.makedirs(path, exist_ok=True)
            return path
    except OSError:
        pass
    path = os.environ.get('MOBULA_JIT_CACHE') or os.path.join(os.path.expanduser('~'), '.cache',
                                                               'mobulaop_amd', 'jit')
    os.makedirs(path, exist_ok=True)
    return path


_INCLUDE = re.compile(r'^[ \t]*#[ \t]*include[ \t]*"([^"]+)"', re.M)


def source_dependencies(source):
    """`source` and every file it includes with #include "...", recursively, looked up
    beside the including file, then in the dialect's and the launcher's include
    directories (what the compiler is given with -I).  The reference walks the same graph
    before it decides to rebuild (mobula/building/build_utils.py: dependant files)."""
    seen, stack = [], [os.path.abspath(source)]
    while stack:
        path = stack.pop()
        if path in seen:
            continue
        seen.append(path)
        try:
            with open(path, 'r', errors='replace') as fin:
                text = fin.read()
        except OSError:
            continue
        for name in _INCLUDE.findall(text):
            for base in (os.path.dirname(path), INC_PATH, CSRC_PATH):
                cand = os.path.normpath(os.path.join(base, name))
                if os.path.isfile(cand):
                    stack.append(cand)
                    break
    return sorted(seen)


def compile_instantiation(cfunc, arg_types, source, symbol):
    """Path of the shared object that exports `symbol`; built if it is not there
    (or was built from another version of the source or of the headers)."""
    build = _build_dir(source)
    # named relative to the build directory where that lies beside the source, so
    # that a tree moved elsewhere finds its shared objects again
    include = os.path.relpath(os.path.abspath(source), build)
    if not include.startswith('..' + os.sep + os.path.basename(source)):
        include = None
    code = wrapper_source(cfunc, arg_types, source, symbol, include)
    digest = hashlib.md5()
    digest.update(code.encode())
    deps = set(source_dependencies(source))
    for header in (os.path.join(INC_PATH, 'mobula_op.h'), os.path.join(INC_PATH, 'mobula_jit.h')):
        deps.update(source_dependencies(header))   # (the wrapper includes these two itself)
    for dep in sorted(deps):
        with open(dep, 'rb') as fin:
            digest.update(fin.read())
    stem = '{}_{}'.format(symbol, digest.hexdigest()[:10])
    lib_path = os.path.join(build, 'lib{}.so'.format(stem))
    if os.path.exists(lib_path):
        return lib_path
    hipcc = shutil.which(config.HIPCC) or '/opt/rocm/bin/hipcc'
    if not os.path.exists(hipcc):
        raise RuntimeError('hipcc not found: {} cannot be compiled'.format(source))
    native.library()   # the wrapper links against the launcher library
    unit = os.path.join(build, stem + '.hip')
    with open(unit, 'w') as fout:
        fout.write(code)
    tmp = lib_path + '.tmp.{}'.format(os.getpid())
    cmd = [hipcc, '--offload-arch=' + config.OFFLOAD_ARCH, '-std=c++17', '-O3', '-fPIC', '-shared',
           '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
           '-I' + INC_PATH, '-I' + CSRC_PATH, '-o', tmp, unit,
           '-L' + CSRC_PATH, '-l:libmobula_hip.so', '-Wl,-rpath,' + CSRC_PATH]
    if config.SHOW_BUILDING_COMMAND:
        print(' '.join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = '\n'.join(l for l in proc.stdout.splitlines()
                    if 'is not a recognized feature for this target' not in l)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise RuntimeError('hipcc failed for {}:\n{}'.format(unit, log))
    os.replace(tmp, lib_path)
    return lib_path


def resolve(cfunc, arg_types, source, symbol):
    """ctypes function `symbol` of the instantiation, compiled on first use."""
    lib_path = compile_instantiation(cfunc, arg_types, source, symbol)
    if lib_path not in _loaded:
        native.library()
        _loaded[lib_path] = ctypes.CDLL(lib_path)
    return getattr(_loaded[lib_path], symbol)
