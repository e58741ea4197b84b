"""The C-ABI library loads without a GPU and exports every symbol that
include/*.h declares; the hashed names are the ones the reference's naming
scheme (mobula/func.py:13-50) yields for the declared argument lists."""
import ctypes
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    names = []
    for header in glob.glob(os.path.join(ROOT, 'include', '*.h')):
        text = re.sub(r'/\*.*?\*/', '', open(header).read(), flags=re.S)
        names += re.findall(r'^\s*(?:const\s+)?[A-Za-z_][\w\s\*]*?\b(\w+)\s*\(', text, flags=re.M)
    return sorted(set(names) - {'defined'})


def test_library_exports_every_declared_symbol():
    from mobulaop_amd import native
    lib = native.library()
    declared = _declared_symbols()
    assert 'roi_align_forward_ab78de3c' in declared and 'roi_align_backward_f318a24e' in declared
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(lib, name), 'library does not export ' + name
    for name in native.exported_names():
        assert hasattr(lib, name), name


def test_symbol_names_follow_the_reference_scheme(mobula):
    from mobulaop_amd.func import get_func_idcode, get_idcode_hash
    from mobulaop_amd.dtype import c_bfloat16, c_half
    # (function, element type T, box type B, symbol); the float and double names are
    # the reference's own (mobula/func.py:13-50 over ROIAlign.cpp:10-16, 79-83)
    cases = [('roi_align_forward', ctypes.c_float, ctypes.c_float, 'roi_align_forward_ab78de3c'),
             ('roi_align_backward', ctypes.c_float, ctypes.c_float, 'roi_align_backward_f318a24e'),
             ('roi_align_forward', ctypes.c_double, ctypes.c_double, 'roi_align_forward_6b9e6c9b'),
             ('roi_align_backward', ctypes.c_double, ctypes.c_double, 'roi_align_backward_2b6c6dfa'),
             ('roi_align_backward_assign', ctypes.c_float, ctypes.c_float,
              'roi_align_backward_assign_a8793cbe'),
             ('roi_align_forward', c_half, ctypes.c_float, 'roi_align_forward_e874c59a'),
             ('roi_align_forward', c_bfloat16, ctypes.c_float, 'roi_align_forward_f951d439'),
             ('roi_align_backward_assign', c_bfloat16, ctypes.c_float, 'roi_align_backward_assign_86156afd')]
    for fname, elem, box, want in cases:
        decl = getattr(mobula.func, fname).func
        bound = {'T': elem, 'B': box}
        types = [t(bound[t.tname]) if hasattr(t, 'tname') else t for t in decl.arg_types]
        assert get_idcode_hash(get_func_idcode(fname, types)) == want


def test_reference_idcode_strings(mobula):
    # the exact strings the reference hashes for the float instantiation
    from mobulaop_amd.func import get_func_idcode
    decl = mobula.func.roi_align_forward.func
    types = [t(ctypes.c_float) if hasattr(t, 'tname') else t for t in decl.arg_types]
    assert get_func_idcode('roi_align_forward', types) == (
        'roi_align_forward:const int,const float*,const float,const int,const int,const int,'
        'const int,const int,const int,const float*,float*')
    decl = mobula.func.roi_align_backward.func
    types = [t(ctypes.c_float) if hasattr(t, 'tname') else t for t in decl.arg_types]
    assert get_func_idcode('roi_align_backward', types) == (
        'roi_align_backward:const int,const float*,const float,const int,const int,const int,'
        'const int,const int,const int,float*,const float*')
    assert decl.arg_names[-2:] == ['bottom_diff', 'bottom_rois']


def test_missing_instantiation_names_the_exports(mobula):
    import numpy as np
    x = np.zeros((1, 1, 2, 2), dtype=np.float64)
    r = np.zeros((1, 5), dtype=np.float32)
    y = np.zeros((1, 1, 1, 1), dtype=np.float64)
    with pytest.raises(NameError) as info:
        mobula.func.roi_align_forward(1, x, 1.0, 1, 2, 2, 1, 1, 1, r, y)
    assert 'roi_align_forward_ab78de3c' in str(info.value)


def test_product_never_imports_the_oracle():
    for path in glob.glob(os.path.join(ROOT, 'mobulaop_amd', '**', '*'), recursive=True):
        if os.path.isfile(path) and path.endswith(('.py', '.hip', '.h')):
            text = open(path).read()
            assert 'oracle' not in text.lower(), path + ' mentions the oracle'
