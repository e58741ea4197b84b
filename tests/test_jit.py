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


# ---------------------------------------------------------------------------
# Kernels whose threads work together, structure arguments, host functions that
# log / check / launch (tests/ops/Reductions, tests/ops/Records).
# ---------------------------------------------------------------------------
class Span(ctypes.Structure):
    _fields_ = [('data', ctypes.POINTER(ctypes.c_float)), ('size', ctypes.c_int)]


class Pair(ctypes.Structure):
    _fields_ = [('count', ctypes.c_int), ('weight', ctypes.c_float)]


def _span_of(tensor):
    """Structure constructor: a view of a float32 tensor of either glue."""
    view = mobula.glue.backend.get_var_glue(tensor).Tensor(tensor)
    ptr = view.data_ptr
    return Span(ctypes.cast(ptr, ctypes.POINTER(ctypes.c_float)), int(view.numel))


@pytest.fixture(scope='module')
def more_ops():
    mobula.glue.register_cstruct('Span', Span, _span_of)
    mobula.glue.register_cstruct('Pair', Pair)
    mobula.op.load('Reductions', OPS)
    mobula.op.load('Records', OPS)
    return mobula.func


_F32P, _F64P, _I32P = (ctypes.POINTER(t) for t in (ctypes.c_float, ctypes.c_double, ctypes.c_int))
_INT = (ctypes.c_int, True)


def _compile(funcs, name, types):
    decl = getattr(funcs, name).func
    symbol = get_idcode_hash(get_func_idcode(name, types))
    source = decl.loader_kwargs['cpp_info'].cpp_fname
    path = jit.compile_instantiation(decl, types, source, symbol)
    assert hasattr(ctypes.CDLL(path), symbol)
    return jit.wrapper_source(decl, types, source, symbol)


def test_synchronising_kernels_are_launched_as_one_workgroup(more_ops):
    # every instantiation the GPU test below calls is compiled here (no GPU needed)
    for ptr in (_F32P, _F64P):
        for name in ('largest', 'plain_total', 'careful_total'):
            code = _compile(more_ops, name, _types(_INT, (ptr, True), (ptr, False)))
            assert 'call.launch_together(' in code
        code = _compile(more_ops, 'row_weights', _types(_INT, _INT, (ptr, True), (ptr, False), (ptr, False)))
        assert 'call.launch_together(' in code
    code = _compile(more_ops, 'contiguous_shares', _types(_INT, (_I32P, False), (_I32P, False)))
    assert 'call.launch_together(' in code
    # a kernel that only uses parfor keeps the many-workgroup launch
    code = _compile(more_ops, 'fill', _types(_INT, (ctypes.c_float, True), (_F32P, False)))
    assert 'call.launch(' in code and 'launch_together' not in code
    # the text scan looks at the kernel's own body, comments excluded
    source = more_ops.largest.func.loader_kwargs['cpp_info'].cpp_fname
    assert jit.synchronises_its_threads(source, 'row_weights_kernel')
    assert 'Reduce' in jit.kernel_body(open(source).read(), 'largest_kernel')
    records = more_ops.fill.func.loader_kwargs['cpp_info'].cpp_fname
    assert not jit.synchronises_its_threads(records, 'fill_kernel')


def test_structures_and_host_functions(more_ops, capfd):
    # symbol names carry `Name*` for a structure, as in the reference (internal/dtype.py:71-74)
    decl = more_ops.span_scale.func
    assert [repr(t) for t in decl.arg_types] == ['const int', 'Span*', 'const float']
    code = _compile(more_ops, 'span_scale', [decl.arg_types[0], decl.arg_types[1], decl.arg_types[2]])
    assert 'call.struct_arg(span)' in code
    # host functions run here: a tuple is spread over the structure's constructor
    assert more_ops.pair_total((3, 0.5)) == 3.5
    assert more_ops.pair_total(Pair(4, 0.25)) == 4.25
    assert 'pair of 3 and 0.5' in capfd.readouterr().out          # LOG(INFO) goes to stdout
    assert more_ops.positive_or_fail(11) == 11
    with pytest.raises(RuntimeError, match='need a positive value'):   # a failed CHECK: an error, not exit()
        more_ops.positive_or_fail(-2)
    assert more_ops.positive_or_fail(5) == 5                           # and the library is usable afterwards
    _compile(more_ops, 'fill_with_sevens', _types(_INT, (_F32P, False)))
    _compile(more_ops, 'round_trip_plus_one', _types(_INT, (_F32P, True), (_F32P, False)))


@pytest.mark.gpu
def test_reductions_run_on_the_gpu(more_ops):
    import math
    import torch
    rng = np.random.default_rng(3)
    for dtype, tol in ((torch.float32, 1e-6), (torch.float64, 1e-15)):
        for n in (1, 63, 1024, 100003):
            xh = rng.standard_normal(n) * 10.0 ** rng.integers(-3, 4, size=n)
            x = torch.from_numpy(xh).to('cuda', dtype)
            out = torch.zeros(4, device='cuda', dtype=dtype)
            more_ops.largest(n, x, out)
            assert float(out[0]) == float(x.max())
            exact = math.fsum(x.double().cpu().tolist())
            scale = float(x.abs().double().sum())
            more_ops.careful_total(n, x, out)
            assert abs(float(out[0]) - exact) <= tol * max(abs(exact), 1e-30) + 4 * tol * scale / max(n, 1) ** 0.5
            more_ops.plain_total(n, x, out)
            assert abs(float(out[0]) - exact) <= 64 * tol * scale
            assert float(out[1]) == 0.0          # only out[0] is written
    x = torch.randn(5, 3001, device='cuda', dtype=torch.float64) * 4
    w = torch.empty_like(x)
    cell = torch.zeros(1, device='cuda', dtype=torch.float64)
    more_ops.row_weights(3001, 5, x, cell, w)
    # against float64 arithmetic on the host (this ROCm build's float64 softmax on the
    # GPU is itself only accurate to ~1e-8)
    xh = x.cpu().numpy()
    e = np.exp(xh - xh.max(axis=1, keepdims=True))
    assert np.abs(w.cpu().numpy() - e / e.sum(axis=1, keepdims=True)).max() <= 1e-15
    owner = torch.full((10007,), -1, device='cuda', dtype=torch.int32)
    threads = torch.zeros(1, device='cuda', dtype=torch.int32)
    more_ops.contiguous_shares(10007, owner, threads)
    t = int(threads[0])
    assert t == 1024
    share, extra = divmod(10007, t)
    want = np.repeat(np.arange(t), [share + (k < extra) for k in range(t)])
    np.testing.assert_array_equal(owner.cpu().numpy(), want)
    # host arrays go through the staging copies like any other kernel
    xh = rng.standard_normal(777).astype(np.float32)
    out = np.zeros(2, dtype=np.float32)
    more_ops.largest(777, xh, out)
    assert out[0] == xh.max()


@pytest.mark.gpu
def test_structures_and_host_launches_on_the_gpu(more_ops):
    import torch
    x = torch.arange(1000, device='cuda', dtype=torch.float32)
    more_ops.span_scale(1, x, 3.0)                     # the constructor builds the Span from the tensor
    assert torch.equal(x, torch.arange(1000, device='cuda', dtype=torch.float32) * 3)
    # a structure that points into ordinary host memory never reaches a kernel
    with pytest.raises(TypeError, match='host memory'):
        more_ops.span_scale(1, np.ones(8, dtype=np.float32), 2.0)
    out = torch.zeros(4099, device='cuda')
    more_ops.fill_with_sevens(out.numel(), out)        # KERNEL_RUN inside a host function
    assert float(out.min()) == 7.0 == float(out.max())
    with pytest.raises(RuntimeError, match='host memory'):
        more_ops.fill_with_sevens(8, np.zeros(8, dtype=np.float32))
    more_ops.fill_with_sevens(out.numel(), out)
    # device memory helpers inside a host function: host arrays in, host arrays out
    src = np.arange(1000, dtype=np.float32)
    dst = np.zeros_like(src)
    assert more_ops.round_trip_plus_one(1000, src, dst) == 1000
    np.testing.assert_array_equal(dst, src + 1)


def test_build_path_configuration(axpy_ops, tmp_path):
    """BUILD_IN_LOCAL_PATH False sends the shared objects to BUILD_PATH/build/<operator>_<hash>/
    (reference behaviour: tests/test_building/test_building.py:47-67)."""
    source = axpy_ops.axpy.func.loader_kwargs['cpp_info'].cpp_fname
    local = jit._build_dir(source)
    assert local == os.path.join(os.path.dirname(source), 'build')
    with mobula.config.TempConfig(BUILD_PATH=str(tmp_path), BUILD_IN_LOCAL_PATH=False):
        moved = jit._build_dir(source)
        assert moved.startswith(os.path.join(str(tmp_path), 'build', 'Axpy_')) and os.path.isdir(moved)
        types = _types((ctypes.c_int, True), (ctypes.c_int, True))
        decl = axpy_ops.padded_length.func
        symbol = get_idcode_hash(get_func_idcode('padded_length', types))
        path = jit.compile_instantiation(decl, types, source, symbol)
        assert os.path.dirname(path) == moved and hasattr(ctypes.CDLL(path), symbol)
    assert jit._build_dir(source) == local


# ---------------------------------------------------------------------------
# Argument kinds of the binding on user kernels (tests/ops/Mixed), mutually
# including files (tests/ops/Loop), rebuilds, failures, concurrent first loads.
# The behaviours are those the reference's own loader tests exercise
# (tests/test_func/test_func.py:44-115, tests/test_building/test_building.py,
# tests/test_parallel/test_multiprocessing.py:21-43).
# ---------------------------------------------------------------------------
@pytest.fixture(scope='module')
def mixed_ops():
    mobula.op.load('Mixed', OPS)
    mobula.op.load('Loop', OPS)
    return mobula.func


def test_host_functions_with_template_return_types_and_include_cycles(mixed_ops):
    assert mixed_ops.loop_answer() == 1234
    for dtype, value in ((np.float32, 5.5), (np.int32, 7), (np.float64, -0.125)):
        src, dst = np.array([value, 1], dtype=dtype), np.zeros(2, dtype=dtype)
        assert mixed_ops.copy_first(src, dst) == value and dst[0] == value and dst[1] == 0


def test_mixed_kernels_compile(mixed_ops):
    f32, i32, f64 = ctypes.c_float, ctypes.c_int, ctypes.c_double
    _compile(mixed_ops, 'five_loops', _types(_INT, *[(_F32P, False)] * 5))
    for scalar in (i32, f32):
        _compile(mixed_ops, 'broadcast', _types(_INT, (scalar, True), (_F32P, False)))
    _compile(mixed_ops, 'fill_like', _types(_INT, (f64, False), (_F64P, False)))
    _compile(mixed_ops, 'address_of', _types(_INT, (ctypes.c_void_p, True),
                                             (ctypes.POINTER(ctypes.c_int64), False)))
    _compile(mixed_ops, 'product_by_atomics', _types(_INT, _INT, _INT, (_F32P, True), (_F32P, True),
                                                     (_F32P, False)))
    code = _compile(mixed_ops, 'ordered_steps', _types(_INT, (_I32P, False), (_I32P, False)))
    assert 'launch_together' in code


def test_a_changed_source_is_rebuilt_and_a_broken_one_reports_the_compiler(tmp_path):
    op_dir = tmp_path / 'Tmp'
    op_dir.mkdir()
    source = op_dir / 'Tmp.cpp'
    source.write_text('MOBULA_FUNC int tmp_value() { return 1; }\n')
    mobula.op.load('Tmp', str(tmp_path))
    decl = mobula.func.tmp_value.func
    first = jit.compile_instantiation(decl, [], str(source), 'tmp_value_d41d8cd9')
    assert ctypes.CDLL(first).tmp_value_d41d8cd9() == 1
    assert jit.compile_instantiation(decl, [], str(source), 'tmp_value_d41d8cd9') == first   # cached
    source.write_text('MOBULA_FUNC int tmp_value() { return 2; }\n')
    second = jit.compile_instantiation(decl, [], str(source), 'tmp_value_d41d8cd9')
    assert second != first and ctypes.CDLL(second).tmp_value_d41d8cd9() == 2
    source.write_text('MOBULA_FUNC int tmp_value() { return not_declared; }\n')
    with pytest.raises(RuntimeError, match='not_declared'):
        jit.compile_instantiation(decl, [], str(source), 'tmp_value_d41d8cd9')
    assert not [f for f in os.listdir(str(op_dir / 'build')) if '.tmp.' in f]   # nothing half-written stays


def test_a_changed_header_of_the_source_is_rebuilt(tmp_path):
    # headers the operator source includes itself are part of what a build is named by
    op_dir = tmp_path / 'Dep'
    op_dir.mkdir()
    (op_dir / 'inner.h').write_text('#define DEP_VALUE 5\n')
    (op_dir / 'outer.h').write_text('#include "inner.h"\n')
    source = op_dir / 'Dep.cpp'
    source.write_text('#include "outer.h"\nMOBULA_FUNC int dep_value() { return DEP_VALUE; }\n')
    deps = jit.source_dependencies(str(source))
    assert [os.path.basename(d) for d in deps] == ['Dep.cpp', 'inner.h', 'outer.h']
    mobula.op.load('Dep', str(tmp_path))
    decl = mobula.func.dep_value.func
    first = jit.compile_instantiation(decl, [], str(source), 'dep_value_d41d8cd9')
    assert ctypes.CDLL(first).dep_value_d41d8cd9() == 5
    (op_dir / 'inner.h').write_text('#define DEP_VALUE 6\n')
    second = jit.compile_instantiation(decl, [], str(source), 'dep_value_d41d8cd9')
    assert second != first and ctypes.CDLL(second).dep_value_d41d8cd9() == 6


_CONCURRENT_LOAD = r'''
import ctypes, os, sys
sys.path.insert(0, sys.argv[1])
import mobulaop_amd as mobula
mobula.config.BUILD_PATH = sys.argv[2]
mobula.config.BUILD_IN_LOCAL_PATH = False
mobula.op.load('Axpy', os.path.join(sys.argv[1], 'tests', 'ops'))
assert mobula.func.padded_length(13, 8) == 16
assert mobula.func.padded_length(16, 8) == 16
print('ok')
'''


def test_processes_loading_the_same_operator_at_once(tmp_path):
    """Several processes build and load one instantiation into an empty build directory at
    the same time: each writes its own temporary file and renames it into place."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = tmp_path / 'load.py'
    script.write_text(_CONCURRENT_LOAD)
    procs = [subprocess.Popen([sys.executable, str(script), root, str(tmp_path / 'shared')],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True) for _ in range(4)]
    outs = [p.communicate(timeout=600)[0] for p in procs]
    assert all(p.returncode == 0 for p in procs), '\n'.join(outs)
    assert all(o.strip().endswith('ok') for o in outs)
    built = [f for d, _, fs in os.walk(str(tmp_path / 'shared')) for f in fs if f.endswith('.so')]
    assert len(built) == 1


@pytest.mark.gpu
def test_mixed_kernels_run_on_the_gpu(mixed_ops):
    import torch
    n = 3000
    outs = [torch.full((m,), -1.0, device='cuda') for m in (n, n // 2, n // 3, 2 * n, 3 * n)]
    mixed_ops.five_loops(n, *outs)
    for out, step in zip(outs, (1, 2, 3, 2, 3)):
        assert torch.equal(out, torch.arange(out.numel(), device='cuda', dtype=torch.float32) * step)
    out = torch.zeros(1000, device='cuda')
    mixed_ops.broadcast(1000, ctypes.c_int(39), out)        # S = int, T = float
    assert float(out.min()) == 39.0 == float(out.max())
    mixed_ops.broadcast(1000, ctypes.c_float(3.5), out)      # S = float
    assert float(out.min()) == 3.5 == float(out.max())
    out64 = torch.zeros(10, device='cuda', dtype=torch.float64)
    mixed_ops.fill_like(10, 0.1, out64)                      # the scalar becomes a double
    assert float(out64[3]) == 0.1
    addr = torch.zeros(4, device='cuda', dtype=torch.int64)
    mixed_ops.address_of(4, ctypes.c_void_p(123456789), addr)
    assert addr.tolist() == [123456789] * 4
    I = U = J = 100
    a, b = torch.rand(I, U, device='cuda'), torch.rand(U, J, device='cuda')
    prod = torch.zeros(I, J, device='cuda')
    mixed_ops.product_by_atomics(U, I, J, a, b, prod)
    want = a.double() @ b.double()
    assert float((prod.double() - want).abs().max()) <= 1e-3
    rounds = 10000
    counter = torch.zeros(1, device='cuda', dtype=torch.int32)
    steps = torch.full((rounds,), -1, device='cuda', dtype=torch.int32)
    mixed_ops.ordered_steps(rounds, counter, steps)
    assert int(counter[0]) == rounds
    assert torch.equal(steps, torch.arange(rounds, device='cuda', dtype=torch.int32))
