"""The convolution oracle against the compiled reference unfold/fold, the
mathematics (fold is the adjoint of unfold) and torch's conv2d on the CPU."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import conv as oracle

CASES = [
    # C, H, W, kernel, pad, stride, dilation
    (2, 3, 4, (2, 3), (0, 1), (1, 2), (1, 1)),      # opzoo/Convolution/test_conv.py:10-14
    (3, 9, 9, (3, 3), (1, 1), (1, 1), (1, 1)),
    (4, 11, 7, (3, 2), (2, 0), (2, 1), (1, 2)),
    (1, 8, 8, (5, 5), (2, 2), (3, 3), (1, 1)),
    (2, 10, 12, (3, 3), (2, 2), (1, 2), (2, 2)),
]


@pytest.mark.parametrize('case', CASES)
def test_unfold_and_fold_match_the_compiled_reference(case):
    if not oracle.ref_available():
        pytest.skip('oracle/_ref/libref_conv.so not built (no reference checkout)')
    C, H, W, kernel, pad, stride, dil = case
    rng = np.random.default_rng(5)
    im = rng.standard_normal((C, H, W)).astype(np.float32)
    col = oracle.im2col(im, kernel, pad, stride, dil)
    assert np.array_equal(col, oracle.im2col(im, kernel, pad, stride, dil, impl='ref'))
    g = rng.standard_normal(col.shape).astype(np.float32)
    back = oracle.col2im(g, im.shape, kernel, pad, stride, dil)
    assert np.array_equal(back, oracle.col2im(g, im.shape, kernel, pad, stride, dil, impl='ref'))


def test_unfold_known_answer():
    # 1x3x3 image, 2x2 window, no padding: four windows, read off by hand
    im = np.arange(9, dtype=np.float32).reshape(1, 3, 3)
    col = oracle.im2col(im, (2, 2), (0, 0), (1, 1), (1, 1))
    want = np.array([[[0, 1], [3, 4]], [[1, 2], [4, 5]], [[3, 4], [6, 7]], [[4, 5], [7, 8]]], np.float32)
    assert np.array_equal(col, want)
    # padding reads zeros
    col = oracle.im2col(im, (1, 1), (1, 1), (1, 1), (1, 1))
    assert col.shape == (1, 5, 5) and col[0, 0].sum() == 0 and np.array_equal(col[0, 1:4, 1:4], im[0])


@pytest.mark.parametrize('case', CASES)
def test_fold_is_the_adjoint_of_unfold(case):
    C, H, W, kernel, pad, stride, dil = case
    rng = np.random.default_rng(6)
    im = rng.standard_normal((C, H, W)).astype(np.float32)
    col = oracle.im2col(im, kernel, pad, stride, dil)
    g = rng.standard_normal(col.shape).astype(np.float32)
    lhs = np.vdot(col.astype(np.float64), g.astype(np.float64))
    rhs = np.vdot(im.astype(np.float64), oracle.col2im(g, im.shape, kernel, pad, stride, dil).astype(np.float64))
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs))


@pytest.mark.parametrize('shape', [
    # N, C, H, W, D, kernel, pad, stride, dilation
    (2, 2, 3, 4, 3, (2, 3), (0, 1), (1, 2), (1, 1)),   # opzoo/Convolution/test_conv.py:10-14
    (3, 4, 9, 8, 6, (3, 3), (1, 1), (1, 1), (1, 1)),
    (2, 3, 12, 10, 5, (3, 2), (2, 1), (2, 1), (1, 2)),
])
def test_convolution_matches_torch(shape):
    N, C, H, W, D, kernel, pad, stride, dil = shape
    g = torch.Generator().manual_seed(11)
    x = torch.randn(N, C, H, W, generator=g, requires_grad=True)
    w = torch.randn(D, C, *kernel, generator=g, requires_grad=True)
    b = torch.randn(D, generator=g, requires_grad=True)
    y = F.conv2d(x, w, b, stride=stride, padding=pad, dilation=dil)
    dy = torch.randn(y.shape, generator=g)
    y.backward(dy)
    got_y = oracle.conv2d_forward(x.detach().numpy(), w.detach().numpy(), b.detach().numpy(), pad, stride, dil)
    dx, dw, db = oracle.conv2d_backward(dy.numpy(), x.detach().numpy(), w.detach().numpy(), pad, stride, dil)
    for got, want in ((got_y, y), (dx, x.grad), (dw, w.grad), (db, b.grad)):
        want = want.detach().numpy()
        assert got.shape == want.shape
        assert np.abs(got - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
