"""Host-side behaviour of the binding, glue and loader (no GPU needed).  The
cases restate what the reference's own tests fix for this boundary:
tests/test_func/test_func.py:9-30 (kwargs, argument checks), tests/test_config.py,
tests/test_testing.py, and the operator/glue contracts of mobula/glue/common.py."""
import ctypes
import os
import textwrap

import numpy as np
import pytest


def test_public_surface(mobula):
    import mobula as alias
    assert alias is mobula
    assert callable(mobula.op.load) and callable(mobula.op.register)
    assert mobula.config.GPU_BACKEND == 'hip'
    for name in ('roi_align_forward', 'roi_align_backward', 'roi_align_backward_assign'):
        assert hasattr(mobula.func, name)
    assert mobula.op.ROIAlign.name == 'ROIAlign'


def test_declaration_scan(tmp_path):
    from mobulaop_amd.op import loader
    from mobulaop_amd.func import CFuncDef
    src = tmp_path / 'Foo.hip'
    src.write_text(textwrap.dedent('''
        template <typename T, typename U>
        MOBULA_KERNEL foo_bar_kernel(const int n, const T* a,
                                     U* out, const U alpha,
                                     void* opaque) { }
        MOBULA_FUNC int64_t plain(const float* p) { return 0; }
    '''))
    funcs = loader._scan_source(str(src))
    foo = funcs['foo_bar']
    assert foo.func_kind == CFuncDef.KERNEL and foo.template_list == ['T', 'U']
    assert foo.arg_names == ['n', 'a', 'out', 'alpha', 'opaque']
    kinds = [(t.is_pointer, t.is_const) for t in foo.arg_types]
    assert kinds == [(False, True), (True, True), (True, False), (False, True), (False, False)]
    assert funcs['plain'].func_kind == CFuncDef.FUNC and funcs['plain'].rtn_type == 'int64_t'
    bad = tmp_path / 'Bad.hip'
    bad.write_text('MOBULA_KERNEL wrong_name(const int n) {}\n')
    with pytest.raises(AssertionError):
        loader._scan_source(str(bad))


def test_load_missing_module(mobula, tmp_path):
    with pytest.raises(AssertionError):
        mobula.op.load('NoSuchOperator', str(tmp_path))


def test_argument_count_and_type_errors(mobula):
    x = np.zeros((1, 1, 2, 2), dtype=np.float32)
    r = np.zeros((1, 5), dtype=np.float32)
    y = np.zeros((1, 1, 1, 1), dtype=np.float32)
    with pytest.raises(KeyError):                                     # too few: missing names
        mobula.func.roi_align_forward(1, x, 1.0)
    with pytest.raises(TypeError):                                    # too many
        mobula.func.roi_align_forward(1, x, 1.0, 1, 2, 2, 1, 1, 1, r, y, 7)
    with pytest.raises(TypeError):
        mobula.func.roi_align_forward(1, [1, 2, 3], 1.0, 1, 2, 2, 1, 1, 1, r, y)  # not a tensor
    with pytest.raises(AssertionError):                               # T bound to float, then double
        mobula.func.roi_align_forward(1, x, 1.0, 1, 2, 2, 1, 1, 1, r, y.astype(np.float64))
    with pytest.raises(NameError):                # float map with double boxes: no such instantiation
        mobula.func.roi_align_forward(1, x, 1.0, 1, 2, 2, 1, 1, 1, r.astype(np.float64), y)
    with pytest.raises(KeyError):                                     # missing keyword
        mobula.func.roi_align_forward(nthreads=1, bottom_data=x)


def test_get_in_data_split():
    from mobulaop_amd.glue.common import get_in_data

    class Op:
        def forward(self, a, b, c=None):
            pass
    inputs, (args, kwargs) = get_in_data(1, 2, 3, 4, k=5, op=Op)
    assert tuple(inputs) == (1, 2, 3) and tuple(args) == (4,) and kwargs == {'k': 5}
    inputs, (args, kwargs) = get_in_data(1, b=2, k=5, op=Op)
    assert list(inputs) == [1, 2] and kwargs == {'k': 5}
    inputs, (args, kwargs) = get_in_data(a=1, b=2, c=3, k=5, op=Op)
    assert list(inputs) == [1, 2, 3] and kwargs == {'k': 5}
    with pytest.raises(AssertionError):
        get_in_data(1, k=5, op=Op)


def test_register_forms_and_numpy_op_object(mobula):
    calls = []

    @mobula.op.register
    class _AddConst:
        def __init__(self, value=1):
            self.value = value

        def forward(self, a):
            calls.append(self.req[0])
            return a + self.value

        def backward(self, dy):
            return dy

        def infer_shape(self, in_shape):
            return in_shape, in_shape
    a = np.arange(4.0)
    op = mobula.op._AddConst[np.ndarray](value=3)
    np.testing.assert_array_equal(op(a), a + 3)
    np.testing.assert_array_equal(op.backward(np.ones(4)), np.ones(4))
    grad = np.full(4, 10.0)
    op.backward(np.ones(4), in_grad=[grad], req=['add'])
    np.testing.assert_array_equal(grad, np.full(4, 11.0))
    np.testing.assert_array_equal(mobula.op._AddConst(a), a + 1)  # default ctor args
    assert calls and all(r == 'write' for r in calls)

    @mobula.op.register('_Renamed', bias=2)
    class _Other:
        def __init__(self, bias):
            self.bias = bias

        def forward(self, a):
            return a * self.bias

        def backward(self, dy):
            return dy * self.bias

        def infer_shape(self, in_shape):
            return in_shape, in_shape
    np.testing.assert_array_equal(mobula.op._Renamed[np.ndarray]()(a), a * 2)


def test_torch_cpu_tensor_goes_through_torch_glue(mobula):
    import torch

    @mobula.op.register
    class _Twice:
        def forward(self, a):
            return a * 2

        def backward(self, dy):
            return dy * 2

        def infer_shape(self, in_shape):
            return in_shape, in_shape
    a = torch.arange(4.0, requires_grad=True)
    out = mobula.op._Twice(a)
    out.sum().backward()
    assert torch.equal(out.detach(), torch.arange(4.0) * 2)
    assert torch.equal(a.grad, torch.full((4,), 2.0))
    with pytest.raises(AssertionError):
        mobula.op._Twice(a, other=np.zeros(3))  # two frameworks in one call


def test_roialign_infer_shape_and_req_null(mobula):
    op = mobula.op.ROIAlign[np.ndarray](pooled_size=(7, 5), spatial_scale=0.5, sampling_ratio=2)
    ins, outs = op.infer_shape([(2, 3, 8, 9), (4, 5)])
    assert outs == [[4, 3, 7, 5]]
    with pytest.raises(AssertionError):
        op.infer_shape([(2, 3, 8, 9), (4, 4)])
    with pytest.raises(AssertionError):
        op.infer_shape([(3, 8, 9), (4, 5)])


def test_config_is_typed(mobula):
    cfg = mobula.config
    with pytest.raises(TypeError):
        cfg.DEBUG = 'yes'
    with pytest.raises(AttributeError):
        cfg.NO_SUCH_KEY = 1
    with cfg.TempConfig(DEBUG=True):
        assert cfg.DEBUG is True
    assert cfg.DEBUG is False
    with pytest.raises(AttributeError):
        with cfg.TempConfig(NO_SUCH_KEY=1):
            pass


def test_assert_almost_equal_criterion(mobula):
    t = mobula.testing
    t.assert_almost_equal(np.array([1.0, 2.0]), np.array([1.0, 2.0 + 1e-9]))
    with pytest.raises(AssertionError):
        t.assert_almost_equal(np.array([1.0]), np.array([1.1]))
    with pytest.raises(AssertionError):          # passes atol, fails rtol
        t.assert_almost_equal(np.array([1e-6]), np.array([2e-6]), rtol=1e-3, atol=1e-3)
    with pytest.raises(AssertionError):
        t.assert_almost_equal(np.zeros(3), np.zeros(4))
    t.assert_parity(np.array([1.0, 1e-9]), np.array([1.0 + 5e-6, 0.0]), 1e-5)
    with pytest.raises(AssertionError):
        t.assert_parity(np.array([1.0, 2e-4]), np.array([1.0, 0.0]), 1e-5)


def test_workloads_are_seeded_and_well_formed():
    from mobulaop_amd import workloads
    a = workloads.make_workload('cfg2', scale_down=64)
    b = workloads.make_workload('cfg2', scale_down=64)
    np.testing.assert_array_equal(a['rois'], b['rois'])
    r = a['rois']
    assert r.shape[1] == 5 and (r[:, 3] > r[:, 1]).all() and (r[:, 4] > r[:, 2]).all()
    assert r[:, 1].min() >= 0 and r[:, 3].max() <= 1344 and r[:, 4].max() <= 800
    w = r[:, 3] - r[:, 1]
    assert w.min() >= 15.9 and w.max() <= 512.1
    full = dict(data=np.empty((4, 256, 200, 336), np.float32), rois=np.empty((4000, 5)),
                pooled_size=(7, 7))
    fwd, bwd = workloads.algorithmic_bytes(full)
    assert abs(fwd - 476.04e6) < 0.05e6 and fwd == bwd
    c3 = workloads.make_workload('cfg3', scale_down=32)
    rr = c3['rois']
    assert ((rr[:, 3] - rr[:, 1]) == 0).any() and (rr[:, 1] < 0).any()
    c4 = workloads.make_workload('cfg4', scale_down=64)
    assert c4['data'].dtype == np.float16 and c4['rois'].dtype == np.float32 and c4['dy'] is None
