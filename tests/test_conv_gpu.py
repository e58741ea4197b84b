"""Parity of the HIP convolution path (through the C-ABI and through the
operator) with the oracle and with torch's conv2d on the CPU.

Tolerance: 1e-3 relative to the largest magnitude of the expected tensor (the
bound the task states for the convolution) for the fp32 products and for the
split-bf16 products (two bf16 per operand, three products); 1e-2 for plain bf16
operands, whose rounding alone (2^-9 per operand) puts a sum of products about
2e-3 off.  im2col / col2im are copies and sums in the reference's order and
must be bit-exact."""
import ctypes

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from mobulaop_amd import native
from oracle import conv as oracle

pytestmark = pytest.mark.gpu
CONV_TOL = 1e-3
# option "conv_compute" -> tolerance
MODES = {'fp32': (0, 1e-3), 'bf16': (1, 1e-2), 'bf16x3': (2, 1e-3)}


@pytest.fixture(params=sorted(MODES))
def compute(request):
    """Runs the test once per way of forming the products; yields the tolerance."""
    mode, tol = MODES[request.param]
    native.set_option('conv_compute', mode)
    yield tol
    native.set_option('conv_compute', 0)


def _ci(*vals):
    return [ctypes.c_int(int(v)) for v in vals]


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _call(name, *args, extents=()):
    lib = native.library()
    native.begin_call(None, list(extents))
    getattr(lib, name)(ctypes.c_int(0), *args)
    native.end_call(name)


def _close(got, want, what, tol=CONV_TOL):
    got, want = got.detach().cpu().double().numpy(), want.detach().cpu().double().numpy()
    assert got.shape == want.shape and np.isfinite(got).all(), what
    err = np.abs(got - want).max()
    assert err <= tol * max(np.abs(want).max(), 1e-30), '{}: max abs error {} vs scale {}'.format(
        what, err, np.abs(want).max())


@pytest.mark.parametrize('case', [
    (2, 3, 4, (2, 3), (0, 1), (1, 2), (1, 1)),
    (5, 17, 13, (3, 3), (1, 1), (1, 1), (1, 1)),
    (3, 20, 16, (3, 2), (2, 0), (2, 1), (1, 2)),
    (2, 12, 12, (3, 3), (2, 2), (1, 2), (2, 2)),
])
def test_unfold_and_fold_bit_exact(case):
    C, H, W, kernel, pad, stride, dil = case
    rng = np.random.default_rng(21)
    im = rng.standard_normal((C, H, W)).astype(np.float32)
    want_col = oracle.im2col(im, kernel, pad, stride, dil)
    OH, OW = want_col.shape[1:]
    geo = _ci(H, W, kernel[0], kernel[1], pad[0], pad[1], stride[0], stride[1], dil[0], dil[1], OH, OW)
    d_im = torch.from_numpy(im).cuda()
    d_col = torch.full(want_col.shape, float('nan'), device='cuda')
    _call('im2col_341af5d3', ctypes.c_int(d_col.numel()), _ptr(d_im), *geo, _ptr(d_col))
    assert np.array_equal(d_col.cpu().numpy(), want_col)
    g = rng.standard_normal(want_col.shape).astype(np.float32)
    d_g = torch.from_numpy(g).cuda()
    d_back = torch.full(im.shape, float('nan'), device='cuda')
    _call('col2im_341af5d3', ctypes.c_int(d_back.numel()), _ptr(d_g), *geo, _ptr(d_back))
    assert np.array_equal(d_back.cpu().numpy(), oracle.col2im(g, im.shape, kernel, pad, stride, dil))


SHAPES = [
    # N, C, H, W, D, kernel, pad, stride, dilation
    (2, 2, 3, 4, 3, (2, 3), (0, 1), (1, 2), (1, 1)),       # opzoo/Convolution/test_conv.py:10-14
    (1, 3, 9, 9, 5, (3, 3), (1, 1), (1, 1), (1, 1)),
    (3, 8, 17, 13, 20, (3, 2), (2, 1), (2, 1), (1, 2)),     # ragged tiles, dilation
    (2, 64, 28, 28, 160, (3, 3), (1, 1), (1, 1), (1, 1)),   # several tiles in every dimension
    (4, 32, 30, 30, 140, (5, 5), (2, 2), (2, 2), (1, 1)),
    (5, 16, 14, 14, 24, (1, 1), (0, 0), (1, 1), (1, 1)),    # pointwise
    (4, 38, 4, 3, 166, (1, 3), (2, 0), (2, 1), (1, 1)),     # 4 x 1 outputs: a step of the weight gradient spans images
    (9, 5, 2, 2, 7, (2, 2), (0, 0), (1, 1), (1, 1)),        # one output pixel per image
]


@pytest.mark.parametrize('shape', SHAPES)
def test_convolution_through_the_abi(shape, compute):
    N, C, H, W, D, kernel, pad, stride, dil = shape
    tol = compute
    g = torch.Generator().manual_seed(31)
    x = torch.randn(N, C, H, W, generator=g)
    w = torch.randn(D, C, *kernel, generator=g) * 0.1
    b = torch.randn(D, generator=g)
    xr, wr, br = (t.clone().requires_grad_(True) for t in (x, w, b))
    y_ref = F.conv2d(xr, wr, br, stride=stride, padding=pad, dilation=dil)
    dy = torch.randn(y_ref.shape, generator=g)
    y_ref.backward(dy)
    if x.numel() * D < 5e6:   # the oracle agrees with torch at sizes it finishes quickly
        y_o = oracle.conv2d_forward(x.numpy(), w.numpy(), b.numpy(), pad, stride, dil)
        assert np.abs(y_o - y_ref.detach().numpy()).max() <= 1e-4 * max(1.0, float(y_ref.detach().abs().max()))
    xd, wd, bd, dyd = x.cuda(), w.cuda(), b.cuda(), dy.cuda()
    geo = _ci(N, C, H, W, D, kernel[0], kernel[1], pad[0], pad[1], stride[0], stride[1], dil[0], dil[1])
    y = torch.full(y_ref.shape, float('nan'), device='cuda')
    _call('conv2d_forward_c6a7aa85', ctypes.c_int(y.numel()), _ptr(xd), _ptr(wd), _ptr(bd), ctypes.c_int(1),
          *geo, _ptr(y))
    _close(y, y_ref, 'y', tol)
    dx = torch.full(x.shape, float('nan'), device='cuda')
    _call('conv2d_backward_data_ecf81c91', ctypes.c_int(dx.numel()), _ptr(dyd), _ptr(wd), ctypes.c_int(0),
          *geo, _ptr(dx))
    _close(dx, xr.grad, 'dx', tol)
    dw = torch.full(w.shape, float('nan'), device='cuda')
    _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw.numel()), _ptr(dyd), _ptr(xd), ctypes.c_int(0),
          *geo, _ptr(dw))
    _close(dw, wr.grad, 'dw', tol)
    db = torch.full((D,), float('nan'), device='cuda')
    _call('conv2d_backward_bias_cd239a08', ctypes.c_int(D), _ptr(dyd), ctypes.c_int(0), ctypes.c_int(N),
          ctypes.c_int(y.shape[2] * y.shape[3]), _ptr(db))
    _close(db, br.grad, 'db', tol)
    # accumulate variants add to what is there
    dx2 = torch.ones_like(dx)
    _call('conv2d_backward_data_ecf81c91', ctypes.c_int(dx2.numel()), _ptr(dyd), _ptr(wd), ctypes.c_int(1),
          *geo, _ptr(dx2))
    _close(dx2 - 1, xr.grad, 'dx accumulate', tol)
    dw2 = torch.ones_like(dw)
    _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw2.numel()), _ptr(dyd), _ptr(xd), ctypes.c_int(1),
          *geo, _ptr(dw2))
    _close(dw2 - 1, wr.grad, 'dw accumulate', tol)


def test_operator_matches_torch_autograd(mobula):
    mobula.op.load('Convolution')
    torch.manual_seed(41)
    x = torch.randn(2, 2, 3, 4, device='cuda', requires_grad=True)       # test_conv.py:10-14
    w = torch.randn(3, 2, 2, 3, device='cuda', requires_grad=True)
    b = torch.randn(3, device='cuda', requires_grad=True)
    y = mobula.op.Conv2D(x=x, weight=w, bias=b, channels=3, kernel_size=(2, 3), strides=(1, 2), padding=(0, 1))
    dy = torch.rand_like(y)
    y.backward(dy)
    xr, wr, br = (t.detach().cpu().requires_grad_(True) for t in (x, w, b))
    yr = F.conv2d(xr, wr, br, stride=(1, 2), padding=(0, 1))
    yr.backward(dy.cpu())
    for got, want, what in ((y, yr, 'y'), (x.grad, xr.grad, 'dx'), (w.grad, wr.grad, 'dw'), (b.grad, br.grad, 'db')):
        _close(got, want, what)
    # without bias
    y2 = mobula.op.Conv2D(x=x.detach(), weight=w.detach(), channels=3, kernel_size=(2, 3), strides=(1, 2),
                          padding=(0, 1))
    _close(y2, F.conv2d(xr.detach(), wr.detach(), None, stride=(1, 2), padding=(0, 1)), 'y without bias')


def test_resnet_block_shape_properties(compute):
    # C_in = C_out = 256, 3x3, pad 1 at a reduced batch and map: linearity in x and
    # the adjoint identity <conv(x), dy> = <x, dx> tie forward and backward together
    N, C, H, W, D = 4, 256, 28, 28, 256
    g = torch.Generator().manual_seed(51)
    x = torch.randn(N, C, H, W, generator=g).cuda()
    w = (torch.randn(D, C, 3, 3, generator=g) * (2.0 / (C * 9)) ** 0.5).cuda()
    dy = torch.randn(N, D, H, W, generator=g).cuda()
    geo = _ci(N, C, H, W, D, 3, 3, 1, 1, 1, 1, 1, 1)
    y = torch.empty(N, D, H, W, device='cuda')
    _call('conv2d_forward_c6a7aa85', ctypes.c_int(y.numel()), _ptr(x), _ptr(w), _ptr(w), ctypes.c_int(0), *geo,
          _ptr(y))
    _close(y, F.conv2d(x.cpu(), w.cpu(), padding=1), 'y', compute)
    dx = torch.empty_like(x)
    _call('conv2d_backward_data_ecf81c91', ctypes.c_int(dx.numel()), _ptr(dy), _ptr(w), ctypes.c_int(0), *geo,
          _ptr(dx))
    dw = torch.empty_like(w)
    _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw.numel()), _ptr(dy), _ptr(x), ctypes.c_int(0), *geo,
          _ptr(dw))
    lhs = float((y.double() * dy.double()).sum())
    if compute <= 1e-3:
        bound = 1e-4 * abs(lhs)
    else:
        # operands rounded to bf16: the three sums round different tensors, and the terms
        # cancel in lhs itself, so the scale is the one of Cauchy-Schwarz
        bound = 1e-3 * float(y.double().norm() * dy.double().norm())
    assert abs(lhs - float((x.double() * dx.double()).sum())) <= bound
    assert abs(lhs - float((w.double() * dw.double()).sum())) <= bound


@pytest.mark.parametrize('mode', ['fp32', 'bf16x3', 'bf16'])
def test_full_cfg5_against_torch(mode):
    # BASELINE configuration 5 at its full size: N=32, 256 -> 256 channels, 56 x 56, 3 x 3,
    # stride 1, pad 1; y, dx and dw against torch's conv2d and its autograd on the CPU, 1e-3
    # (1e-2 with operands rounded to bf16)
    N, C, H, W, D = 32, 256, 56, 56, 256
    g = torch.Generator().manual_seed(1005)
    xh = torch.randn(N, C, H, W, generator=g)
    wh = torch.randn(D, C, 3, 3, generator=g) * (2.0 / (C * 9)) ** 0.5   # Kaiming-normal
    dyh = torch.randn(N, D, H, W, generator=g)
    xr, wr = xh.clone().requires_grad_(True), wh.clone().requires_grad_(True)
    print('cfg5: torch conv2d on the CPU ...', flush=True)
    yr = F.conv2d(xr, wr, padding=1)
    yr.backward(dyh)
    native.set_option('conv_compute', MODES[mode][0])
    try:
        x, w, dy = xh.cuda(), wh.cuda(), dyh.cuda()
        geo = _ci(N, C, H, W, D, 3, 3, 1, 1, 1, 1, 1, 1)
        y = torch.empty(N, D, H, W, device='cuda')
        _call('conv2d_forward_c6a7aa85', ctypes.c_int(y.numel()), _ptr(x), _ptr(w), _ptr(w), ctypes.c_int(0), *geo,
              _ptr(y))
        _close(y, yr, 'cfg5 y ' + mode, MODES[mode][1])
        dx = torch.empty_like(x)
        _call('conv2d_backward_data_ecf81c91', ctypes.c_int(dx.numel()), _ptr(dy), _ptr(w), ctypes.c_int(0), *geo,
              _ptr(dx))
        _close(dx, xr.grad, 'cfg5 dx ' + mode, MODES[mode][1])
        dw = torch.empty_like(w)
        _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw.numel()), _ptr(dy), _ptr(x), ctypes.c_int(0),
              *geo, _ptr(dw))
        _close(dw, wr.grad, 'cfg5 dw ' + mode, MODES[mode][1])
    finally:
        native.set_option('conv_compute', 0)


@pytest.mark.parametrize('shape', [
    # N, C, H, W, D, kernel, pad, stride, dilation
    (3, 40, 24, 24, 72, (3, 3), (1, 1), (1, 1), (1, 1)),    # rows of four: the 16-byte conversion
    (2, 33, 19, 21, 50, (3, 2), (2, 0), (1, 1), (1, 1)),    # odd rows: the element-wise conversion
    (4, 64, 56, 56, 64, (3, 3), (1, 1), (1, 1), (1, 1)),    # planes longer than one conversion span
    (1, 3, 12, 12, 5, (3, 3), (1, 1), (1, 1), (1, 1)),      # N * C odd: the sets of planes end off a 256-byte boundary
    (3, 5, 9, 11, 7, (3, 3), (1, 1), (1, 1), (1, 1)),       # likewise with an odd grid width
    (1, 4, 70, 71, 6, (3, 3), (1, 1), (1, 1), (1, 1)),      # the element-wise conversion over planes of two spans
    (3, 8, 17, 13, 20, (3, 2), (2, 1), (2, 1), (1, 2)),     # strides and dilation: the gathered weight gradient
    (4, 32, 30, 30, 140, (5, 5), (2, 2), (2, 2), (1, 1)),   # several channel blocks and row tiles, strides
    (2, 70, 23, 17, 200, (3, 3), (1, 1), (1, 1), (1, 1)),   # channels not a multiple of 32
])
def test_split_operands_keep_every_cross_term(shape):
    # Two bf16 per fp32 and three products (head x head, head x tail, tail x head) leave errors of
    # about 2^-16 of the operands; leaving out one cross term would leave about 2^-9, the error
    # of operands rounded to bf16.  Reference: the same sums in float64.
    N, C, H, W, D, kernel, pad, stride, dil = shape
    g = torch.Generator().manual_seed(77)
    x = torch.randn(N, C, H, W, generator=g)
    w = torch.randn(D, C, *kernel, generator=g) * 0.1
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    y_ref = F.conv2d(xr, wr, None, stride=stride, padding=pad, dilation=dil)
    dy = torch.randn(y_ref.shape, generator=g)
    y_ref.backward(dy.double())
    try:
        native.set_option('conv_compute', 1)
        _leave_nan_patterns_in_the_workspace()
        native.set_option('conv_compute', 2)
        xd, wd, dyd = x.cuda(), w.cuda(), dy.cuda()
        geo = _ci(N, C, H, W, D, kernel[0], kernel[1], pad[0], pad[1], stride[0], stride[1], dil[0], dil[1])
        y = torch.full(y_ref.shape, float('nan'), device='cuda')
        _call('conv2d_forward_c6a7aa85', ctypes.c_int(y.numel()), _ptr(xd), _ptr(wd), _ptr(wd), ctypes.c_int(0),
              *geo, _ptr(y))
        _close(y, y_ref, 'y', 3e-5)
        dx = torch.full(x.shape, float('nan'), device='cuda')
        _call('conv2d_backward_data_ecf81c91', ctypes.c_int(dx.numel()), _ptr(dyd), _ptr(wd), ctypes.c_int(0),
              *geo, _ptr(dx))
        _close(dx, xr.grad, 'dx', 3e-5)
        dw = torch.full(w.shape, float('nan'), device='cuda')
        _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw.numel()), _ptr(dyd), _ptr(xd), ctypes.c_int(0),
              *geo, _ptr(dw))
        _close(dw, wr.grad, 'dw', 3e-5)
    finally:
        native.set_option('conv_compute', 0)


def test_random_shapes_in_every_mode():
    # sixty seeded shapes (channel counts around the 32-channel blocks, strides, dilation, padding
    # beyond the kernel, widths with and without 16-byte rows), each in one of the three ways of
    # forming the products, against torch's float64 convolution and its autograd
    tol = {0: 2e-5, 2: 3e-5}
    done = 0
    for case in range(80):
        rng = np.random.default_rng(5000 + case)
        N, C, D = int(rng.integers(1, 5)), int(rng.choice([1, 3, 8, 31, 32, 33, 64, 70])), int(rng.choice([1, 5, 32, 100, 129, 260]))
        H, W = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        if rng.integers(0, 2):
            W = (W + 3) // 4 * 4
        kh, kw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        ph, pw = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        sh, sw = (1, 1) if rng.integers(0, 3) else (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        dh, dw_ = (1, 1) if rng.integers(0, 3) else (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        mode = int(rng.integers(0, 3))
        if H + 2 * ph < dh * (kh - 1) + 1 or W + 2 * pw < dw_ * (kw - 1) + 1:
            continue
        g = torch.Generator().manual_seed(5000 + case)
        x = torch.randn(N, C, H, W, generator=g)
        w = torch.randn(D, C, kh, kw, generator=g) * 0.2
        xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
        y_ref = F.conv2d(xr, wr, None, stride=(sh, sw), padding=(ph, pw), dilation=(dh, dw_))
        dy = torch.randn(y_ref.shape, generator=g)
        y_ref.backward(dy.double())
        what = 'case {}: mode {} N{} C{} {}x{} D{} k{}x{} p{},{} s{},{} d{},{}'.format(
            case, mode, N, C, H, W, D, kh, kw, ph, pw, sh, sw, dh, dw_)
        print(what, flush=True)
        native.set_option('conv_compute', mode)
        try:
            xd, wd, dyd = x.cuda(), w.cuda(), dy.cuda()
            geo = _ci(N, C, H, W, D, kh, kw, ph, pw, sh, sw, dh, dw_)
            y = torch.full(y_ref.shape, float('nan'), device='cuda')
            _call('conv2d_forward_c6a7aa85', ctypes.c_int(y.numel()), _ptr(xd), _ptr(wd), _ptr(wd), ctypes.c_int(0),
                  *geo, _ptr(y))
            dx = torch.full(x.shape, float('nan'), device='cuda')
            _call('conv2d_backward_data_ecf81c91', ctypes.c_int(dx.numel()), _ptr(dyd), _ptr(wd), ctypes.c_int(0),
                  *geo, _ptr(dx))
            dw = torch.full(w.shape, float('nan'), device='cuda')
            _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw.numel()), _ptr(dyd), _ptr(xd), ctypes.c_int(0),
                  *geo, _ptr(dw))
        finally:
            native.set_option('conv_compute', 0)
        if mode == 1:
            # operands rounded to bf16 are off by up to 2^-9 each: the bound is a share of the sum of
            # the terms' magnitudes, which a sum that cancels can be far below
            xa, wa = x.double().abs().requires_grad_(True), w.double().abs().requires_grad_(True)
            ya = F.conv2d(xa, wa, None, stride=(sh, sw), padding=(ph, pw), dilation=(dh, dw_))
            ya.backward(dy.double().abs())
            for got, want, mag, name in ((y, y_ref, ya, ' y'), (dx, xr.grad, xa.grad, ' dx'), (dw, wr.grad, wa.grad, ' dw')):
                err = float((got.cpu().double() - want.detach()).abs().max())
                assert err <= 2.0 ** -7 * float(mag.detach().max()), what + name
        else:
            _close(y, y_ref, what + ' y', tol[mode])
            _close(dx, xr.grad, what + ' dx', tol[mode])
            _close(dw, wr.grad, what + ' dw', tol[mode])
        done += 1
    assert done >= 60


def _leave_nan_patterns_in_the_workspace():
    # The bf16 products keep copies of their operands in the calling thread's workspace, which
    # is not cleared between calls: a product of NaN inputs (conv_compute must be 1) leaves NaN
    # bit patterns behind, so a later call that read bytes it had not written itself would show.
    x = torch.full((2, 32, 40, 40), float('nan'), device='cuda')
    w = torch.full((32, 32, 3, 3), float('nan'), device='cuda')
    y = torch.empty(2, 32, 40, 40, device='cuda')
    geo = _ci(2, 32, 40, 40, 32, 3, 3, 1, 1, 1, 1, 1, 1)
    _call('conv2d_forward_c6a7aa85', ctypes.c_int(y.numel()), _ptr(x), _ptr(w), _ptr(w), ctypes.c_int(0), *geo,
          _ptr(y))
    dw = torch.empty_like(w)
    _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw.numel()), _ptr(y), _ptr(x), ctypes.c_int(0), *geo,
          _ptr(dw))
    torch.cuda.synchronize()


@pytest.mark.parametrize('case', [
    # N, C, H, W, D, kernel, pad, stride, dilation
    (3, 64, 20, 20, 96, (3, 3), (1, 1), (1, 1), (1, 1)),      # 128-row tiles
    (2, 70, 23, 17, 200, (3, 3), (1, 1), (1, 1), (1, 1)),     # 256-row tiles, channels not a multiple of 32
    (2, 40, 19, 21, 130, (5, 3), (2, 0), (1, 1), (1, 2)),     # dilation, uneven padding
    (2, 33, 30, 26, 300, (3, 3), (1, 1), (2, 2), (1, 1)),     # strides: two row tiles, gathered weight gradient
    (9, 256, 28, 28, 256, (3, 3), (1, 1), (1, 1), (1, 1)),    # several images to a tile, K cut into pieces
    (1, 16, 60, 60, 16, (1, 1), (0, 0), (1, 1), (1, 1)),      # one tap
    (2, 8, 96, 96, 12, (3, 3), (1, 1), (1, 1), (1, 1)),       # planes of several spans in the padded copies
    (1, 8, 70, 104, 8, (1, 3), (0, 1), (1, 1), (1, 1)),       # likewise, no padded rows
    (1, 3, 12, 12, 5, (3, 3), (1, 1), (1, 1), (1, 1)),        # N * C odd: the padded copies end off a 256-byte boundary
    (3, 5, 9, 11, 7, (3, 3), (1, 1), (1, 1), (1, 1)),         # likewise, odd grid width (the scalar copy)
    (2, 20, 20, 20, 100, (3, 3), (1, 1), (1, 1), (1, 1)),     # 128-row tiles with channels not a multiple of 32
    (1, 6, 21, 20, 9, (1, 2), (0, 0), (1, 1), (1, 1)),        # an odd shift without padding
    (1, 4, 70, 71, 6, (3, 3), (1, 1), (1, 1), (1, 1)),        # odd width: the scalar copy over planes of two spans
    (1, 2, 3, 4100, 4, (3, 3), (1, 1), (1, 1), (1, 1)),       # grid rows longer than a span
])
def test_bf16_mode_is_exact_on_bf16_valued_operands(case):
    # Mode 1 rounds both operands of every product to bf16 and accumulates in fp32: against
    # the same products of the rounded operands in fp32 only the order of the sums differs,
    # well inside the 1e-3 bound (the 1e-2 of the other tests is the rounding of the inputs)
    N, C, H, W, D, k, pad, stride, dil = case
    g = torch.Generator().manual_seed(61)
    x = torch.randn(N, C, H, W, generator=g)
    w = torch.randn(D, C, *k, generator=g) * 0.1
    rnd = lambda t: t.bfloat16().float()
    xr, wr = rnd(x).requires_grad_(True), rnd(w).requires_grad_(True)
    yr = F.conv2d(xr, wr, padding=pad, stride=stride, dilation=dil)
    dy = torch.randn(yr.shape, generator=g)
    yr.backward(rnd(dy))
    native.set_option('conv_compute', 1)
    try:
        _leave_nan_patterns_in_the_workspace()
        xd, wd, dyd = x.cuda(), w.cuda(), dy.cuda()
        geo = _ci(N, C, H, W, D, k[0], k[1], pad[0], pad[1], stride[0], stride[1], dil[0], dil[1])
        y = torch.empty(yr.shape, device='cuda')
        _call('conv2d_forward_c6a7aa85', ctypes.c_int(y.numel()), _ptr(xd), _ptr(wd), _ptr(wd), ctypes.c_int(0),
              *geo, _ptr(y))
        dx = torch.empty_like(xd)
        _call('conv2d_backward_data_ecf81c91', ctypes.c_int(dx.numel()), _ptr(dyd), _ptr(wd), ctypes.c_int(0),
              *geo, _ptr(dx))
        dw = torch.empty_like(wd)
        _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw.numel()), _ptr(dyd), _ptr(xd), ctypes.c_int(0),
              *geo, _ptr(dw))
        # accumulate: twice the gradient on top of what is there
        dw2 = dw.clone()
        _call('conv2d_backward_weight_ecf81c91', ctypes.c_int(dw.numel()), _ptr(dyd), _ptr(xd), ctypes.c_int(1),
              *geo, _ptr(dw2))
        dx2 = dx.clone()
        _call('conv2d_backward_data_ecf81c91', ctypes.c_int(dx.numel()), _ptr(dyd), _ptr(wd), ctypes.c_int(1),
              *geo, _ptr(dx2))
    finally:
        native.set_option('conv_compute', 0)
    _close(y, yr.detach(), 'y', 1e-4)
    _close(dx, xr.grad, 'dx', 1e-4)
    _close(dw, wr.grad, 'dw', 1e-4)
    _close(dw2, 2 * wr.grad, 'dw accumulated', 1e-4)
    _close(dx2, 2 * xr.grad, 'dx accumulated', 1e-4)


def test_errors_surface_as_exceptions():
    x = torch.zeros(1, 1, 4, 4, device='cuda')
    w = torch.zeros(1, 1, 3, 3, device='cuda')
    y = torch.zeros(1, 1, 2, 2, device='cuda')
    geo = _ci(1, 1, 4, 4, 1, 3, 3, 0, 0, 1, 1, 1, 1)
    with pytest.raises(RuntimeError):   # wrong output element count
        _call('conv2d_forward_c6a7aa85', ctypes.c_int(3), _ptr(x), _ptr(w), _ptr(w), ctypes.c_int(0), *geo, _ptr(y))
    with pytest.raises(RuntimeError):   # window larger than the padded input
        _call('conv2d_forward_c6a7aa85', ctypes.c_int(4), _ptr(x), _ptr(w), _ptr(w), ctypes.c_int(0),
              *_ci(1, 1, 2, 2, 1, 3, 3, 0, 0, 1, 1, 1, 1), _ptr(y))
    lib = native.library()
    native.begin_call(None, [])
    lib.conv2d_forward_c6a7aa85(ctypes.c_int(-1), ctypes.c_int(4), _ptr(x), _ptr(w), _ptr(w), ctypes.c_int(0), *geo,
                                _ptr(y))
    with pytest.raises(RuntimeError):   # host buffers are not staged for the convolution
        native.end_call('conv2d_forward')
    # the library stays usable
    _call('conv2d_forward_c6a7aa85', ctypes.c_int(4), _ptr(x), _ptr(w), _ptr(w), ctypes.c_int(0), *geo, _ptr(y))
