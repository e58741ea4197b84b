"""Compile-on-load of a user operator written in MobulaOP's kernel dialect
(tests/ops/Axpy): code generation and compilation here, execution on the GPU."""
import ctypes
import os

import numpy as np
import pytest

import mobulaop_amd as mobula
from mobulaop_amd.dtype import DType
from mobulaop_amd.func import get_func_idcode, get_idcode_hash
from mobulaop_amd.op import jit

OPS = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'ops')


@pytest.fixture(scope='module')
def axpy_ops():
    mobula.op.load('Axpy', OPS)
    return mobula.func


def _types(*spec):
    return [DType(t, is_const=c) for t, c in spec]


def test_wrapper_names_the_symbol_like_the_reference(axpy_ops):
    # axpy<float>: const int, const float, const float*, float*
    decl = axpy_ops.axpy.func
    types = _types((ctypes.c_int, True), (ctypes.c_float, True), (ctypes.POINTER(ctypes.c_float), True),
                   (ctypes.POINTER(ctypes.c_float), False))
    symbol = get_idcode_hash(get_func_idcode('axpy', types))
    assert symbol.startswith('axpy_') and len(symbol) == len('axpy_') + 8
    code = jit.wrapper_source(decl, types, decl.loader_kwargs['cpp_info'].cpp_fname, symbol)
    assert 'void {}(const int device_id, const int n, const float a, const float* x, float* y)'.format(symbol) in code
    assert 'axpy_kernel<float>' in code and 'call.arg(y, 3, true)' in code and 'call.arg(x, 2, false)' in code


def test_instantiations_compile_and_export_their_symbols(axpy_ops):
    # no GPU needed: hipcc cross-compiles, the shared object is only inspected
    for scalar in (ctypes.c_float, ctypes.c_double):
        decl = axpy_ops.axpy.func
        types = _types((ctypes.c_int, True), (scalar, True), (ctypes.POINTER(scalar), True),
                       (ctypes.POINTER(scalar), False))
        symbol = get_idcode_hash(get_func_idcode('axpy', types))
        path = jit.compile_instantiation(decl, types, decl.loader_kwargs['cpp_info'].cpp_fname, symbol)
        assert os.path.exists(path)
        assert hasattr(ctypes.CDLL(path), symbol)
    # the other kernels of the source, as the GPU tests call them
    f32p, i32p = ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_int)
    for name, types in (
            ('weighted_histogram', _types((ctypes.c_int, True), (i32p, True), (f32p, True), (f32p, False))),
            ('row_energy', _types((ctypes.c_int, True), (ctypes.c_int, True), (f32p, True), (f32p, False)))):
        decl = getattr(axpy_ops, name).func
        symbol = get_idcode_hash(get_func_idcode(name, types))
        path = jit.compile_instantiation(decl, types, decl.loader_kwargs['cpp_info'].cpp_fname, symbol)
        assert hasattr(ctypes.CDLL(path), symbol)
    assert axpy_ops.padded_length(13, 8) == 16      # MOBULA_FUNC: runs on the host


@pytest.mark.gpu
def test_user_kernels_run_on_torch_tensors(axpy_ops):
    import torch
    for dtype in (torch.float32, torch.float64):
        x = torch.randn(100003, device='cuda', dtype=dtype)
        y = torch.randn(100003, device='cuda', dtype=dtype)
        want = y + 2.5 * x
        axpy_ops.axpy(x.numel(), 2.5, x, y)
        assert float((y - want).abs().max()) <= 1e-6 * float(want.abs().max())
    bins = torch.randint(0, 7, (50000,), device='cuda', dtype=torch.int32)
    w = torch.rand(50000, device='cuda')
    hist = torch.zeros(7, device='cuda')
    axpy_ops.weighted_histogram(bins.numel(), bins, w, hist)
    want = torch.zeros(7, device='cuda').index_add_(0, bins.long(), w)
    # fp32 sums of 7000 terms in two different orders
    assert float((hist - want).abs().max()) <= 1e-5 * float(want.abs().max())
    x = torch.randn(300, 17, device='cuda')
    out = torch.empty(300, device='cuda')
    axpy_ops.row_energy(300, 17, x, out)
    assert float((out - (x * x).sum(1)).abs().max()) <= 1e-4


@pytest.mark.gpu
def test_user_kernel_on_host_arrays_is_staged_through_the_gpu(axpy_ops):
    x = np.arange(1000, dtype=np.float32)
    y = np.ones(1000, dtype=np.float32)
    axpy_ops.axpy(x.size, np.float32(0.5), x, y)
    assert np.allclose(y, 1 + 0.5 * x)


@pytest.mark.gpu
def test_user_operator_class_through_autograd(axpy_ops):
    import torch
    x = torch.randn(4, 5, device='cuda', requires_grad=True)
    b = torch.randn(4, 5, device='cuda', requires_grad=True)
    y = mobula.op.Axpy(x, b, a=3.0)
    assert float((y - (3 * x + b)).detach().abs().max()) <= 1e-6
    y.backward(torch.ones_like(y))
    assert float((x.grad - 3).abs().max()) <= 1e-6 and float((b.grad - 1).abs().max()) <= 1e-6


def test_build_directory_is_never_created_in_a_read_only_source_tree(tmp_path, monkeypatch):
    """A source directory without the owner's write bit is left alone even when the
    process could write there (root): the shared objects go to the cache instead."""
    import stat
    from mobulaop_amd.op import jit
    src_dir = tmp_path / 'readonly' / 'Op'
    src_dir.mkdir(parents=True)
    (src_dir / 'Op.cpp').write_text('// empty\n')
    src_dir.chmod(stat.S_IRUSR | stat.S_IXUSR | stat.S_IRGRP | stat.S_IXGRP)
    monkeypatch.setenv('MOBULA_JIT_CACHE', str(tmp_path / 'cache'))
    try:
        chosen = jit._build_dir(str(src_dir / 'Op.cpp'))
        assert chosen == str(tmp_path / 'cache')
        assert not (src_dir / 'build').exists()
    finally:
        src_dir.chmod(stat.S_IRWXU)
    # a writable source directory still gets its build/ beside the source
    assert jit._build_dir(str(src_dir / 'Op.cpp')) == str(src_dir / 'build')
