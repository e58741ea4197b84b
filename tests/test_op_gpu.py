"""GPU tests of the Python surface: `mobula.op.ROIAlign` through the torch and
NumPy glues and `mobula.func.*` directly, checked against the CPU oracle."""
import numpy as np
import pytest

torch = pytest.importorskip('torch')

from mobulaop_amd import workloads  # noqa: E402
from mobulaop_amd.testing import assert_parity  # noqa: E402
from oracle import roialign as oracle  # noqa: E402

pytestmark = pytest.mark.gpu
FWD_TOL, BWD_TOL = 1e-5, 1e-4


@pytest.fixture(autouse=True)
def _announce(request):
    print('\n[case] {}'.format(request.node.nodeid), flush=True)


def _small():
    w = workloads.make_workload('cfg2', scale_down=32)
    want_y = oracle.forward(w['data'], w['rois'], w['pooled_size'], w['spatial_scale'],
                            w['sampling_ratio'])
    want_dx = oracle.backward(w['dy'], w['rois'], w['data'].shape, w['spatial_scale'],
                              w['sampling_ratio'], impl='ordered')
    return w, want_y, want_dx


def test_reference_example_through_torch(mobula):
    # examples/RunROIAlign.py:12-26 with torch tensors on the GPU
    x = torch.arange(2 * 3 * 4 * 4, dtype=torch.float32, device='cuda').reshape(2, 3, 4, 4)
    x.requires_grad_(True)
    rois = torch.tensor([[0, 1, 1, 3, 3]], dtype=torch.float32, device='cuda')
    out = mobula.op.ROIAlign(data=x, rois=rois, pooled_size=(2, 2), spatial_scale=1.0,
                             sampling_ratio=1)
    out.backward(torch.ones_like(out))
    want = torch.tensor([[7.5, 8.5], [11.5, 12.5]], device='cuda')
    for c in range(3):
        assert torch.equal(out[0, c].detach(), want + 16 * c)
    k = torch.tensor([[.25, .5, .25], [.5, 1, .5], [.25, .5, .25]], device='cuda')
    assert torch.equal(x.grad[0, 0, 1:4, 1:4], k) and float(x.grad[1].abs().sum()) == 0


def test_torch_autograd_path(mobula):
    w, want_y, want_dx = _small()
    x = torch.from_numpy(w['data']).cuda().requires_grad_(True)
    rois = torch.from_numpy(w['rois']).cuda().requires_grad_(True)
    y = mobula.op.ROIAlign(x, rois, pooled_size=w['pooled_size'],
                           spatial_scale=w['spatial_scale'], sampling_ratio=w['sampling_ratio'])
    assert y.requires_grad and y.shape == want_y.shape
    y.backward(torch.from_numpy(w['dy']).cuda())
    assert_parity(y, want_y, FWD_TOL, 'y')
    assert_parity(x.grad, want_dx, BWD_TOL, 'dx')
    assert float(rois.grad.abs().max()) == 0      # no gradient to the boxes
    # a second backward accumulates into .grad exactly once
    y2 = mobula.op.ROIAlign(x, rois, pooled_size=w['pooled_size'],
                            spatial_scale=w['spatial_scale'], sampling_ratio=w['sampling_ratio'])
    y2.backward(torch.from_numpy(w['dy']).cuda())
    assert_parity(x.grad, 2 * want_dx, BWD_TOL, 'dx twice')


def test_numpy_path_stages_through_the_gpu(mobula):
    w, want_y, want_dx = _small()
    op = mobula.op.ROIAlign[np.ndarray](pooled_size=w['pooled_size'],
                                        spatial_scale=w['spatial_scale'],
                                        sampling_ratio=w['sampling_ratio'])
    y = op(w['data'], w['rois'])
    assert isinstance(y, np.ndarray)
    assert_parity(y, want_y, FWD_TOL, 'y')
    dx, drois = op.backward(w['dy'])
    assert_parity(dx, want_dx, BWD_TOL, 'dx')
    assert not drois.any()
    # req = add accumulates into the caller's gradient, req = null leaves it alone
    base = np.ones_like(w['data'])
    op.backward(w['dy'], in_grad=[base, np.zeros_like(w['rois'])], req=['add', 'null'])
    assert_parity(base, want_dx + 1, BWD_TOL, 'dx add')


def test_direct_function_calls_kwargs_and_strided_tensors(mobula):
    w, want_y, want_dx = _small()
    N, C, H, W = w['data'].shape
    PH, PW = w['pooled_size']
    x = torch.from_numpy(w['data']).cuda()
    rois = torch.from_numpy(w['rois']).cuda()
    # output written through a non-contiguous view: copied back after the call
    backing = torch.zeros(want_y.shape[0], C, PH, 2 * PW, device='cuda')
    y_view = backing[..., ::2]
    assert not y_view.is_contiguous()
    mobula.func.roi_align_forward(
        nthreads=y_view.numel(), bottom_data=x, spatial_scale=w['spatial_scale'], channels=C,
        height=H, width=W, pooled_height=PH, pooled_width=PW, sampling_ratio=w['sampling_ratio'],
        bottom_rois=rois, top_data=y_view)
    assert_parity(backing[..., ::2], want_y, FWD_TOL, 'strided y')
    assert float(backing[..., 1::2].abs().sum()) == 0
    # strided input
    x_t = torch.from_numpy(np.ascontiguousarray(w['data'].transpose(0, 1, 3, 2))).cuda().transpose(2, 3)
    assert not x_t.is_contiguous()
    y = torch.empty(want_y.shape, device='cuda')
    mobula.func.roi_align_forward(y.numel(), x_t, w['spatial_scale'], C, H, W, PH, PW,
                                  w['sampling_ratio'], rois, y)
    assert_parity(y, want_y, FWD_TOL, 'strided x')
    dx = torch.zeros(N, C, H, W, device='cuda')
    mobula.func.roi_align_backward(y.numel(), torch.from_numpy(w['dy']).cuda(), w['spatial_scale'],
                                   C, H, W, PH, PW, w['sampling_ratio'], dx, rois)
    assert_parity(dx, want_dx, BWD_TOL, 'dx')


def test_errors_surface_as_python_exceptions(mobula):
    x = torch.rand(1, 2, 4, 4, device='cuda')
    rois = torch.zeros(2, 5, device='cuda')
    y = torch.empty(3, 2, 2, 2, device='cuda')  # claims 3 ROIs, rois has 2
    with pytest.raises(RuntimeError):
        mobula.func.roi_align_forward(y.numel(), x, 1.0, 2, 4, 4, 2, 2, 2, rois, y)
    with pytest.raises(AssertionError):          # host and device tensor in one call
        mobula.func.roi_align_forward(8, x, 1.0, 2, 4, 4, 2, 2, 2, rois.cpu().numpy(), y)


def test_runs_on_the_callers_stream(mobula):
    w, want_y, _ = _small()
    x = torch.from_numpy(w['data']).cuda()
    rois = torch.from_numpy(w['rois']).cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        y = mobula.op.ROIAlign(x, rois, pooled_size=w['pooled_size'],
                               spatial_scale=w['spatial_scale'],
                               sampling_ratio=w['sampling_ratio'])
        doubled = y * 2          # ordered after the kernel on the same stream
    side.synchronize()
    assert_parity(doubled, 2 * want_y, FWD_TOL, 'stream')


def test_channels_last_tensors_take_the_channels_last_path(mobula):
    # same numbers as with NCHW tensors; outputs and gradients come back channels-last
    torch.manual_seed(5)
    x = torch.randn(2, 32, 20, 24, device='cuda')
    rois = torch.tensor([[0, 1, 2, 60, 50], [1, 10, 10, 90, 70], [1, -5, 3, 20, 100]], device='cuda',
                        dtype=torch.float32)
    kw = dict(pooled_size=(7, 7), spatial_scale=0.25, sampling_ratio=2)
    xa = x.clone().requires_grad_(True)
    ya = mobula.op.ROIAlign(xa, rois, **kw)
    dy = torch.randn_like(ya)
    ya.backward(dy)
    xb = x.clone().to(memory_format=torch.channels_last).requires_grad_(True)
    yb = mobula.op.ROIAlign(xb, rois, **kw)
    assert yb.is_contiguous(memory_format=torch.channels_last) and not yb.is_contiguous()
    yb.backward(dy)
    assert xb.grad.is_contiguous(memory_format=torch.channels_last)
    assert float((ya - yb).detach().abs().max()) <= 1e-5 * float(ya.detach().abs().max())
    assert float((xa.grad - xb.grad).abs().max()) <= 1e-4 * float(xa.grad.abs().max())


@pytest.mark.parametrize('low,tol', [(torch.float16, 2e-3), (torch.bfloat16, 8e-3)])
def test_half_precision_training_step(mobula, low, tol):
    # 16-bit map and gradients through the operator: both passes run in the library
    # (bfloat16 carries 8 significant bits: 4e-3 per rounding)
    torch.manual_seed(6)
    x32 = torch.randn(2, 64, 20, 24, device='cuda')
    rois = torch.tensor([[0, 1, 2, 60, 50], [1, 10, 10, 90, 70], [1, -5, 3, 20, 100]], device='cuda',
                        dtype=torch.float32)
    kw = dict(pooled_size=(7, 7), spatial_scale=0.25, sampling_ratio=2)
    xh = x32.to(low).requires_grad_(True)
    yh = mobula.op.ROIAlign(xh, rois, **kw)
    assert yh.dtype == low
    dy = torch.randn_like(yh)
    yh.backward(dy)
    assert xh.grad.dtype == low
    xf = x32.to(low).float().requires_grad_(True)
    yf = mobula.op.ROIAlign(xf, rois, **kw)
    yf.backward(dy.float())
    assert float((yh.detach().float() - yf.detach()).abs().max()) <= tol * float(yf.detach().abs().max())
    assert float((xh.grad.float() - xf.grad).abs().max()) <= tol * float(xf.grad.abs().max())
    # channels-last 16-bit maps: the forward reads them where they lie
    xc = x32.to(low).contiguous(memory_format=torch.channels_last)
    xc.requires_grad_(True)
    yc = mobula.op.ROIAlign(xc, rois, **kw)
    assert float((yc.detach().float() - yf.detach()).abs().max()) <= tol * float(yf.detach().abs().max())
    yc.backward(dy.contiguous(memory_format=torch.channels_last))
    assert xc.grad.dtype == low and xc.grad.is_contiguous(memory_format=torch.channels_last)
    assert float((xc.grad.float() - xf.grad).abs().max()) <= tol * float(xf.grad.abs().max())


def test_double_tensors_through_the_operator(mobula):
    """float64 data and boxes resolve to the double instantiation; autograd gets dx."""
    rng = np.random.default_rng(9)
    xh = rng.standard_normal((2, 3, 12, 14))
    rh = np.array([[0, 2.5, 3.5, 30.25, 28.0], [1, -4, 0, 20, 44], [1, 8, 8, 8, 8]], dtype=np.float64)
    dyh = rng.standard_normal((3, 3, 4, 4))
    x = torch.from_numpy(xh).cuda().requires_grad_(True)
    rois = torch.from_numpy(rh).cuda()
    y = mobula.op.ROIAlign(x, rois, pooled_size=(4, 4), spatial_scale=0.25, sampling_ratio=0)
    assert y.dtype == torch.float64
    np.testing.assert_array_equal(y.detach().cpu().numpy(), oracle.forward_f64(xh, rh, (4, 4), 0.25, 0))
    y.backward(torch.from_numpy(dyh).cuda())
    np.testing.assert_allclose(x.grad.cpu().numpy(), oracle.backward_f64(dyh, rh, xh.shape, 0.25, 0),
                               rtol=0, atol=1e-13)
    # host arrays take the same symbols (device id -1: staged through the GPU)
    out = np.zeros((3, 3, 4, 4))
    mobula.func.roi_align_forward(out.size, xh, 0.25, 3, 12, 14, 4, 4, 0, rh, out)
    np.testing.assert_array_equal(out, oracle.forward_f64(xh, rh, (4, 4), 0.25, 0))
