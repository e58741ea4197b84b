"""Pins for the CPU oracle (oracle/roialign_oracle.c): none of these re-types the
oracle's formula.  They are (1) the compiled reference kernels (oracle/_ref, built
from the reference sources where those exist), (2) the closed-form case of the
reference's own example (examples/RunROIAlign.py:12-26), (3) plane invariance,
(4) the adjoint identity, (5) an independent NumPy loop, (6) committed golden
fixtures, (7) the edge semantics of bilinear.h:15-44."""
import os

import numpy as np
import pytest

from oracle import roialign as oracle

GOLDEN = os.path.join(os.path.dirname(__file__), 'golden')


def _random_case(rng, N=3, C=4, H=13, W=17, R=9, pooled=(3, 4), scale=0.25, span=80.0):
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    c = rng.uniform(-5, span, size=(R, 2))
    wh = rng.uniform(0, span, size=(R, 2))
    b = rng.integers(0, N, size=(R, 1))
    rois = np.concatenate([b, c - wh / 2, c + wh / 2], axis=1).astype(np.float32)
    dy = rng.standard_normal((R, C) + pooled).astype(np.float32)
    return x, rois, dy, pooled, scale


def test_known_answer_from_reference_example():
    # x = arange, roi [0,1,1,3,3], 2x2, scale 1, S=1 -> samples at pixel centres 1.5, 2.5
    x = np.arange(2 * 3 * 4 * 4, dtype=np.float32).reshape(2, 3, 4, 4)
    rois = np.array([[0, 1, 1, 3, 3]], dtype=np.float32)
    y = oracle.forward(x, rois, (2, 2), 1.0, 1)
    want = np.array([[7.5, 8.5], [11.5, 12.5]], dtype=np.float32)
    for c in range(3):
        np.testing.assert_array_equal(y[0, c], want + 16 * c)
    dx = oracle.backward(np.ones_like(y), rois, x.shape, 1.0, 1)
    k = np.array([[.25, .5, .25], [.5, 1, .5], [.25, .5, .25]], dtype=np.float32)
    want_dx = np.zeros_like(x)
    want_dx[0, :, 1:4, 1:4] = k
    np.testing.assert_array_equal(dx, want_dx)
    assert dx[1].sum() == 0


def test_plane_is_reproduced_at_bin_centres():
    # bilinear interpolation is exact on a*y + b*x + c, and the sampling grid is
    # symmetric about the bin centre, so the output is the plane at the centre
    H = W = 12
    yy, xx = np.mgrid[0:H, 0:W].astype(np.float32)
    x = (3 * yy + 2 * xx + 1)[None, None]
    rois = np.array([[0, 1, 1, 5, 5], [0, 2.5, 0.5, 9.0, 10.0]], dtype=np.float32)
    for S in (1, 2, 3):
        y = oracle.forward(x, rois, (2, 2), 1.0, S)
        np.testing.assert_allclose(y[0, 0], [[11, 15], [17, 21]], rtol=1e-6)
        x1, y1, x2, y2 = rois[1, 1:]
        cy = y1 + (np.arange(2) + .5) * (y2 - y1) / 2
        cx = x1 + (np.arange(2) + .5) * (x2 - x1) / 2
        np.testing.assert_allclose(y[1, 0], 3 * cy[:, None] + 2 * cx[None, :] + 1, rtol=1e-6)


@pytest.mark.parametrize('S', [0, 1, 2, 3])
def test_adjoint_identity(S):
    # the operator is linear in x: <fwd(x), dy> == <x, bwd(dy)>
    rng = np.random.default_rng(7 + S)
    x, rois, dy, pooled, scale = _random_case(rng)
    y = oracle.forward(x, rois, pooled, scale, S)
    dx = oracle.backward(dy, rois, x.shape, scale, S, impl='ordered')
    lhs = np.sum(y.astype(np.float64) * dy)
    rhs = np.sum(x.astype(np.float64) * dx)
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs))


@pytest.mark.parametrize('S', [0, 2])
def test_against_independent_numpy_loop(S):
    rng = np.random.default_rng(11 + S)
    x, rois, dy, pooled, scale = _random_case(rng, N=2, C=2, H=9, W=11, R=5, span=50.0)
    y_bf, dx_bf = oracle.brute_force(x, rois, pooled, scale, S, dy)
    y = oracle.forward(x, rois, pooled, scale, S)
    dx = oracle.backward(dy, rois, x.shape, scale, S, impl='ordered')
    # same samples and weights; only the association of the 4-term sum differs
    np.testing.assert_allclose(y, y_bf, rtol=2e-6, atol=2e-6)
    np.testing.assert_allclose(dx, dx_bf, rtol=2e-5, atol=2e-6)


def test_reference_test_configuration():
    # the shape of the reference's own value test (opzoo/ROIAlign/test_roialign.py:243-282):
    # N,C,H,W = 5,3,16,16, R=7, pooled (3,4), scale 16/224, S=0, data = arange
    rng = np.random.default_rng(5)
    N, C, H, W, R = 5, 3, 16, 16, 7
    x = np.arange(N * C * H * W, dtype=np.float32).reshape(N, C, H, W)
    c = rng.uniform(0, 224, size=(R, 2))
    wh = rng.uniform(0, 224, size=(R, 2))
    rois = np.concatenate([rng.integers(0, N, size=(R, 1)), c - wh / 2, c + wh / 2],
                          axis=1).astype(np.float32)
    dy = rng.uniform(-1, 1, size=(R, C, 3, 4)).astype(np.float32)
    y_bf, dx_bf = oracle.brute_force(x, rois, (3, 4), 16 / 224, 0, dy)
    y = oracle.forward(x, rois, (3, 4), 16 / 224, 0)
    dx = oracle.backward(dy, rois, x.shape, 16 / 224, 0)
    # the reference's own tolerance for this case is atol = rtol = 1e-3
    np.testing.assert_allclose(y, y_bf, rtol=1e-5, atol=1e-3)
    np.testing.assert_allclose(dx, dx_bf, rtol=1e-4, atol=1e-4)


def test_edge_semantics():
    H = W = 8
    x = np.arange(H * W, dtype=np.float32).reshape(1, 1, H, W) + 1
    f = lambda roi, S=1, pooled=(1, 1): oracle.forward(
        x, np.array([roi], dtype=np.float32), pooled, 1.0, S)[0, 0]
    # zero-width / reversed boxes are forced to 1x1 anchored at the start corner
    np.testing.assert_array_equal(f([0, 2, 3, 2, 3]), f([0, 2, 3, 3, 4]))
    np.testing.assert_array_equal(f([0, 2, 3, 1, 1]), f([0, 2, 3, 3, 4]))
    # sample at (2.5, 3.5): mean of the 2x2 block at rows 3..4, cols 2..3
    assert f([0, 2, 3, 3, 4])[0, 0] == x[0, 0, 3:5, 2:4].mean()
    # entirely outside the map
    assert f([0, 100, 100, 120, 120])[0, 0] == 0
    assert f([0, -50, -50, -40, -40])[0, 0] == 0
    # a sample exactly at y == H still counts (clamped to the last row) ...
    at_edge = f([0, 0, 7.5, 1, 8.5])[0, 0]      # centre y = 8.0 = H, x = 0.5
    assert at_edge == (x[0, 0, 7, 0] + x[0, 0, 7, 1]) / 2
    # ... while anything above H contributes nothing
    assert f([0, 0, 7.75, 1, 8.75])[0, 0] == 0
    # y in [-1, 0] clamps to row 0 and counts
    assert f([0, 0, -1.25, 1, -0.25])[0, 0] == (x[0, 0, 0, 0] + x[0, 0, 0, 1]) / 2
    assert f([0, 0, -2.5, 1, -1.5])[0, 0] == 0
    # adaptive grid: ceil(roi/pooled) samples per bin and axis.  On a constant map
    # the output is (#valid samples)/count: a 5x6 box hanging 4 rows above the map
    # has sample rows -3.5 ... 1.5, of which 3 of 6 are >= -1
    ones = np.ones((1, 1, H, W), dtype=np.float32)
    box = np.array([[0, 0, -4, 5, 2]], dtype=np.float32)
    assert oracle.forward(ones, box, (1, 1), 1.0, 0)[0, 0, 0, 0] == 0.5
    assert oracle.forward(ones, box, (1, 1), 1.0, 1)[0, 0, 0, 0] == 1.0   # one sample at y = -1
    assert oracle.forward(ones, box, (1, 1), 1.0, 2)[0, 0, 0, 0] == 0.5   # rows -2.5 and 0.5
    # batch index is truncated toward zero
    x2 = np.concatenate([x, x + 100], axis=0)
    r = np.array([[0.9, 2, 3, 3, 4], [1.9, 2, 3, 3, 4]], dtype=np.float32)
    y2 = oracle.forward(x2, r, (1, 1), 1.0, 1)
    assert y2[0, 0, 0, 0] + 100 == y2[1, 0, 0, 0]


needs_ref = pytest.mark.skipif(not oracle.ref_available('serial'),
                               reason='oracle/_ref not built (reference checkout absent)')


@needs_ref
@pytest.mark.parametrize('S', [0, 1, 2])
def test_bit_exact_against_compiled_reference(S):
    rng = np.random.default_rng(100 + S)
    x, rois, dy, pooled, scale = _random_case(rng, N=3, C=5, H=20, W=27, R=40, span=140.0)
    # add adversarial boxes: outside, zero-size, sub-pixel
    rois[0, 1:] = [200, 200, 260, 260]
    rois[1, 1:] = [10, 10, 10, 10]
    rois[2, 1:] = [33.3, 20.1, 33.6, 20.2]
    rois[3, 1:] = [-30, -30, 50, 20]
    for impl in ('ref_omp', 'ref_serial'):
        np.testing.assert_array_equal(oracle.forward(x, rois, pooled, scale, S),
                                      oracle.forward(x, rois, pooled, scale, S, impl=impl))
    # fixed-order backward == single-thread reference, bit for bit
    np.testing.assert_array_equal(
        oracle.backward(dy, rois, x.shape, scale, S, impl='ordered'),
        oracle.backward(dy, rois, x.shape, scale, S, impl='ref_serial'))
    # the atomic schedule differs only by summation order
    a = oracle.backward(dy, rois, x.shape, scale, S)
    b = oracle.backward(dy, rois, x.shape, scale, S, impl='ref_omp')
    np.testing.assert_allclose(a, b, rtol=0, atol=1e-5)


def test_golden_fixtures():
    files = sorted(f for f in os.listdir(GOLDEN) if f.endswith('.npz'))
    assert files, 'no golden fixtures committed'
    for name in files:
        z = np.load(os.path.join(GOLDEN, name))
        pooled = tuple(int(v) for v in z['pooled_size'])
        scale, S = float(z['spatial_scale']), int(z['sampling_ratio'])
        y = oracle.forward(z['data'], z['rois'], pooled, scale, S)
        np.testing.assert_array_equal(y, z['y'], err_msg=name)
        dx = oracle.backward(z['dy'], z['rois'], z['data'].shape, scale, S, impl='ordered')
        np.testing.assert_array_equal(dx, z['dx'], err_msg=name)


# ---------------------------------------------------------------------------
# The double instantiation (oracle/roialign_oracle_f64.c).
# ---------------------------------------------------------------------------
def _random_case_f64(rng, **kw):
    x, rois, dy, pooled, scale = _random_case(rng, **kw)
    # fresh float64 draws (not widened float32 values): every mantissa bit in play
    return (x + 1e-9 * rng.standard_normal(x.shape), rois.astype(np.float64) + 1e-7 * rng.random(rois.shape)
            * (np.arange(5) > 0), dy + 1e-9 * rng.standard_normal(dy.shape), pooled, scale)


def test_f64_known_answer_and_plane():
    x = np.arange(2 * 3 * 4 * 4, dtype=np.float64).reshape(2, 3, 4, 4)
    rois = np.array([[0, 1, 1, 3, 3]], dtype=np.float64)
    y = oracle.forward_f64(x, rois, (2, 2), 1.0, 1)
    for c in range(3):
        np.testing.assert_array_equal(y[0, c], np.array([[7.5, 8.5], [11.5, 12.5]]) + 16 * c)
    dx = oracle.backward_f64(np.ones_like(y), rois, x.shape, 1.0, 1)
    want = np.zeros_like(x)
    want[0, :, 1:4, 1:4] = [[.25, .5, .25], [.5, 1, .5], [.25, .5, .25]]
    np.testing.assert_array_equal(dx, want)
    # a plane a*y + b*x + c is reproduced at the bin centres when every sample is inside
    H, W = 12, 15
    yy, xx = np.mgrid[0:H, 0:W]
    plane = (3.0 * yy + 2.0 * xx + 1.0)[None, None]
    out = oracle.forward_f64(plane, np.array([[0, 1, 1, 5, 5]], dtype=np.float64), (2, 2), 1.0, 2)
    np.testing.assert_allclose(out[0, 0], [[11, 15], [17, 21]], rtol=1e-14)


@pytest.mark.parametrize('S', [0, 1, 2, 3])
def test_f64_against_independent_numpy_loop_and_adjoint(S):
    rng = np.random.default_rng(300 + S)
    x, rois, dy, pooled, scale = _random_case_f64(rng, N=2, C=2, H=9, W=11, R=6, span=50.0)
    rois[0, 1:] = [-20, -20, 15, 10]      # partly outside
    rois[1, 1:] = [12, 12, 12, 12]        # zero size
    y = oracle.forward_f64(x, rois, pooled, scale, S)
    dx = oracle.backward_f64(dy, rois, x.shape, scale, S)
    want_y, want_dx = oracle.brute_force(x, rois, pooled, scale, S, dy=dy, dtype=np.float64)
    np.testing.assert_array_equal(y, want_y)
    np.testing.assert_allclose(dx, want_dx, rtol=0, atol=1e-14)
    # the operator is linear in x: <fwd(x), dy> == <x, bwd(dy)>
    lhs, rhs = float((y * dy).sum()), float((x * dx).sum())
    assert abs(lhs - rhs) <= 1e-12 * max(1.0, np.abs(y * dy).sum())
    # and genuinely double: the float32 kernels differ from it at float32 precision only
    y32 = oracle.forward(x, rois, pooled, scale, S)
    assert 0 < np.abs(y32 - y).max() < 1e-4


@needs_ref
@pytest.mark.parametrize('S', [0, 2])
def test_f64_bit_exact_against_compiled_reference(S):
    rng = np.random.default_rng(400 + S)
    x, rois, _, pooled, scale = _random_case_f64(rng, N=3, C=3, H=20, W=27, R=30, span=140.0)
    rois[0, 1:] = [200, 200, 260, 260]
    rois[1, 1:] = [10, 10, 10, 10]
    rois[2, 1:] = [33.3, 20.1, 33.6, 20.2]
    rois[3, 1:] = [-30, -30, 50, 20]
    for impl in ('ref_omp', 'ref_serial'):
        np.testing.assert_array_equal(oracle.forward_f64(x, rois, pooled, scale, S),
                                      oracle.forward_f64(x, rois, pooled, scale, S, impl=impl))


def test_f64_golden_fixtures():
    folder = os.path.join(GOLDEN, 'f64')
    files = sorted(f for f in os.listdir(folder) if f.endswith('.npz'))
    assert files, 'no double fixtures committed'
    for name in files:
        z = np.load(os.path.join(folder, name))
        pooled = tuple(int(v) for v in z['pooled_size'])
        y = oracle.forward_f64(z['data'], z['rois'], pooled, float(z['spatial_scale']),
                               int(z['sampling_ratio']))
        np.testing.assert_array_equal(y, z['y'], err_msg=name)
