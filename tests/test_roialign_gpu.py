"""GPU parity tests: the HIP kernels, called through the C ABI, against the CPU
oracle and the committed golden vectors on the same seeded inputs.

Tolerances (stated by the task for this path): forward 1e-5, backward 1e-4
(atomic / tile summation order differs), fp16 storage 2e-3; gated both
elementwise (|a-b| <= tol * max(|b|, max|b|)) and as ||a-b||_inf <= tol * ||b||_inf
(mobulaop_amd/testing.py: assert_parity).
"""
import os

import numpy as np
import pytest

torch = pytest.importorskip('torch')

from mobulaop_amd import native, workloads  # noqa: E402
from mobulaop_amd.testing import assert_parity  # noqa: E402
from oracle import roialign as oracle  # noqa: E402
import abi_util as abi  # noqa: E402

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), 'golden')
FWD_TOL, BWD_TOL, FP16_TOL = 1e-5, 1e-4, 2e-3
IMPLS = ['naive', 'tiled']


@pytest.fixture(autouse=True)
def _announce(request):
    print('\n[case] {}'.format(request.node.nodeid), flush=True)
    yield
    abi.set_impl('auto')
    native.set_option('roialign_tile_columns', 0)
    native.set_option('roialign_row_split', 0)
    native.set_option('roialign_row_quads', 1)


@pytest.mark.parametrize('impl', IMPLS)
def test_golden_vectors(impl):
    abi.set_impl(impl)
    for name in sorted(f for f in os.listdir(GOLDEN) if f.endswith('.npz')):
        z = np.load(os.path.join(GOLDEN, name))
        pooled = tuple(int(v) for v in z['pooled_size'])
        scale, S = float(z['spatial_scale']), int(z['sampling_ratio'])
        x, rois, dy = abi.to_dev(z['data']), abi.to_dev(z['rois']), abi.to_dev(z['dy'])
        y = abi.forward(x, rois, pooled, scale, S).cpu().numpy()
        assert_parity(y, z['y'], FWD_TOL, name + ' fwd')
        dx = abi.backward(dy, rois, x.shape, scale, S).cpu().numpy()
        assert_parity(dx, z['dx'], BWD_TOL, name + ' bwd')
        dx2 = abi.backward(dy, rois, x.shape, scale, S, assign=True).cpu().numpy()
        assert_parity(dx2, z['dx'], BWD_TOL, name + ' bwd assign')


@pytest.mark.skipif(not oracle.ref_available('serial'), reason='oracle/_ref is not built')
def test_golden_inputs_against_the_compiled_reference():
    # the compiled reference kernels themselves (oracle/_ref, built in the development
    # container from the reference's sources) as the checker, where they travelled along
    for name in sorted(f for f in os.listdir(GOLDEN) if f.endswith('.npz')):
        z = np.load(os.path.join(GOLDEN, name))
        pooled = tuple(int(v) for v in z['pooled_size'])
        scale, S = float(z['spatial_scale']), int(z['sampling_ratio'])
        x, rois, dy = abi.to_dev(z['data']), abi.to_dev(z['rois']), abi.to_dev(z['dy'])
        want_y = oracle.forward(z['data'], z['rois'], pooled, scale, S, impl='ref_serial')
        assert_parity(abi.forward(x, rois, pooled, scale, S).cpu().numpy(), want_y, FWD_TOL, name + ' fwd vs _ref')
        want_dx = oracle.backward(z['dy'], z['rois'], z['data'].shape, scale, S, impl='ref_serial')
        assert_parity(abi.backward(dy, rois, x.shape, scale, S).cpu().numpy(), want_dx, BWD_TOL,
                      name + ' bwd vs _ref')


def test_full_cfg1_against_oracle():
    # the reference's own CPU-runnable configuration at its full size, every element
    w = workloads.make_workload('cfg1')
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    x, rois, dy = abi.to_dev(w['data']), abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    y = abi.forward(x, rois, pooled, scale, S).cpu().numpy()
    assert_parity(y, oracle.forward(w['data'], w['rois'], pooled, scale, S), FWD_TOL, 'cfg1 fwd')
    want_dx = oracle.backward(w['dy'], w['rois'], w['data'].shape, scale, S, impl='ordered')
    assert_parity(abi.backward(dy, rois, x.shape, scale, S).cpu().numpy(), want_dx, BWD_TOL, 'cfg1 bwd')
    assert_parity(abi.backward(dy, rois, x.shape, scale, S, assign=True).cpu().numpy(), want_dx, BWD_TOL,
                  'cfg1 bwd assign')


@pytest.mark.parametrize('impl', IMPLS)
@pytest.mark.parametrize('cfg,down', [('cfg1', 8), ('cfg2', 16), ('cfg3', 32)])
def test_scaled_configs_against_oracle(impl, cfg, down):
    abi.set_impl(impl)
    w = workloads.make_workload(cfg, scale_down=down)
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    x, rois, dy = abi.to_dev(w['data']), abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    y = abi.forward(x, rois, pooled, scale, S).cpu().numpy()
    assert_parity(y, oracle.forward(w['data'], w['rois'], pooled, scale, S), FWD_TOL, cfg + ' fwd')
    want_dx = oracle.backward(w['dy'], w['rois'], w['data'].shape, scale, S, impl='ordered')
    dx = abi.backward(dy, rois, x.shape, scale, S).cpu().numpy()
    assert_parity(dx, want_dx, BWD_TOL, cfg + ' bwd')
    dx = abi.backward(dy, rois, x.shape, scale, S, assign=True).cpu().numpy()
    assert_parity(dx, want_dx, BWD_TOL, cfg + ' bwd assign')


def test_tiled_backward_repeats_bit_for_bit():
    """The tiled backward owns every dx element in one wavefront and adds in list
    order (no float atomics), so two runs agree exactly; the reference's
    atomics (ROIAlign.cpp:149-156) give a few ulp of run-to-run noise."""
    abi.set_impl('tiled')
    w = workloads.make_workload('cfg3', scale_down=16)   # heavy overlap, adversarial boxes
    scale, S = w['spatial_scale'], w['sampling_ratio']
    rois, dy = abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    first = abi.backward(dy, rois, w['data'].shape, scale, S, assign=True)
    for _ in range(3):
        again = abi.backward(dy, rois, w['data'].shape, scale, S, assign=True)
        assert torch.equal(first, again)


@pytest.mark.parametrize('impl', IMPLS)
def test_backward_accumulates_into_existing_gradient(impl):
    abi.set_impl(impl)
    w = workloads.make_workload('cfg1', scale_down=16)
    scale, S = w['spatial_scale'], w['sampling_ratio']
    rois, dy = abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    base = np.random.default_rng(3).standard_normal(w['data'].shape).astype(np.float32)
    dx = abi.backward(dy, rois, base.shape, scale, S, dx=abi.to_dev(base)).cpu().numpy()
    want = oracle.backward(w['dy'], w['rois'], base.shape, scale, S, impl='ordered', dx=base.copy())
    assert_parity(dx, want, BWD_TOL, 'accumulate')


@pytest.mark.parametrize('impl', IMPLS)
def test_fp16_storage_forward(impl):
    abi.set_impl(impl)
    w = workloads.make_workload('cfg4', scale_down=16)
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    x16 = w['data']
    y = abi.forward(abi.to_dev(x16), abi.to_dev(w['rois']), pooled, scale, S).cpu().numpy()
    assert y.dtype == np.float16
    want = oracle.forward(x16.astype(np.float32), w['rois'], pooled, scale, S)
    assert_parity(y.astype(np.float32), want.astype(np.float16).astype(np.float32), FP16_TOL, 'fp16')


@pytest.mark.parametrize('S', [2, 0, 3])
@pytest.mark.parametrize('C', [72, 64, 20])
def test_fp16_channel_blocks(C, S):
    # fp16 maps are blocked by 64 channels, eight per lane: a ragged last block (72), exact
    # blocks (64), and a count that is no multiple of eight (20: straightforward kernel)
    abi.set_impl('auto')
    rng = np.random.default_rng(100 * C + S)
    N, H, W, R, pooled, scale = 2, 30, 44, 60, (7, 7), 0.25
    x16 = rng.standard_normal((N, C, H, W)).astype(np.float16)
    c = np.stack([rng.uniform(0, W / scale, R), rng.uniform(0, H / scale, R)], 1)
    wh = np.stack([rng.uniform(2, W / scale, R), rng.uniform(2, H / scale, R)], 1)
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    y = abi.forward(abi.to_dev(x16), abi.to_dev(rois), pooled, scale, S).cpu().numpy()
    assert y.dtype == np.float16
    want = oracle.forward(x16.astype(np.float32), rois, pooled, scale, S)
    assert_parity(y.astype(np.float32), want.astype(np.float16).astype(np.float32), FP16_TOL, 'fp16')


BF16_TOL = 4e-3   # a bfloat16 result carries 8 significant bits: half a unit in the last place is 2e-3


def _round_bf16(a):
    """float32 array -> the nearest bfloat16 values, as float32 (round to nearest even)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).float().numpy()


@pytest.mark.parametrize('S', [2, 0])
@pytest.mark.parametrize('C', [72, 64, 20])
def test_bfloat16_storage(C, S):
    """bfloat16 maps and gradients (fp32 boxes, fp32 arithmetic): the checker's fp32 result on
    the bfloat16-rounded operands, rounded to bfloat16.  NCHW and channels-last; C = 20 and the
    S = 0 backward go through the straightforward kernels."""
    abi.set_impl('auto')
    rng = np.random.default_rng(500 * C + S)
    N, H, W, R, pooled, scale = 2, 30, 44, 50, (7, 7), 0.25
    xb = _round_bf16(rng.standard_normal((N, C, H, W)))
    dyb = _round_bf16(rng.standard_normal((R, C) + pooled))
    c = np.stack([rng.uniform(0, W / scale, R), rng.uniform(0, H / scale, R)], 1)
    wh = np.stack([rng.uniform(2, W / scale, R), rng.uniform(2, H / scale, R)], 1)
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    x = abi.to_dev(xb).to(torch.bfloat16)
    dy = abi.to_dev(dyb).to(torch.bfloat16)
    r = abi.to_dev(rois)
    want_y = _round_bf16(oracle.forward(xb, rois, pooled, scale, S))
    y = abi.forward(x, r, pooled, scale, S)
    assert y.dtype == torch.bfloat16
    assert_parity(y.float().cpu().numpy(), want_y, BF16_TOL, 'bf16 fwd')
    if C % 8 == 0:
        y_cl = abi.forward_nhwc(x.permute(0, 2, 3, 1).contiguous(), r, pooled, scale, S)
        assert_parity(y_cl.permute(0, 3, 1, 2).float().cpu().numpy(), want_y, BF16_TOL, 'bf16 fwd channels-last')
    want_dx = oracle.backward(dyb, rois, (N, C, H, W), scale, S, impl='ordered')
    dx = abi.backward(dy, r, (N, C, H, W), scale, S, assign=True)
    assert dx.dtype == torch.bfloat16
    assert_parity(dx.float().cpu().numpy(), _round_bf16(want_dx), BF16_TOL, 'bf16 bwd assign')
    base = _round_bf16(rng.standard_normal((N, C, H, W)))
    dx = abi.backward(dy, r, (N, C, H, W), scale, S, dx=abi.to_dev(base).to(torch.bfloat16))
    assert_parity(dx.float().cpu().numpy(), _round_bf16(want_dx + base), BF16_TOL, 'bf16 bwd accumulate')
    if native.roialign_channels_last_supported(True, 2, C, H, W, pooled, S, R):
        # channels-last gradients of both 16-bit types, overwriting and accumulating
        for low, rnd, tol in ((torch.bfloat16, _round_bf16, BF16_TOL),
                              (torch.float16, lambda a: a.astype(np.float16).astype(np.float32), FP16_TOL)):
            dy_cl = abi.to_dev(dyb).to(low).permute(0, 2, 3, 1).contiguous()
            want = oracle.backward(dy_cl.permute(0, 3, 1, 2).float().cpu().numpy(), rois, (N, C, H, W), scale, S,
                                   impl='ordered')
            got = abi.backward_nhwc(dy_cl, r, (N, H, W, C), scale, S, assign=True)
            assert got.dtype == low
            assert_parity(got.permute(0, 3, 1, 2).float().cpu().numpy(), rnd(want), tol, 'channels-last bwd assign')
            seed = abi.to_dev(base).to(low).permute(0, 2, 3, 1).contiguous()
            want_acc = want + seed.permute(0, 3, 1, 2).float().cpu().numpy()
            got = abi.backward_nhwc(dy_cl, r, (N, H, W, C), scale, S, dx=seed)
            assert_parity(got.permute(0, 3, 1, 2).float().cpu().numpy(), rnd(want_acc), tol,
                          'channels-last bwd accumulate')


@pytest.mark.parametrize('S', [2, 0])
@pytest.mark.parametrize('C', [72, 20])
def test_fp16_backward(C, S):
    # fp16 gradients: the checker's fp32 result on the fp16-rounded dy, rounded to fp16;
    # S = 0 (and C = 20 in any case) goes through the straightforward kernel and an fp32 scratch map
    abi.set_impl('auto')
    rng = np.random.default_rng(300 * C + S)
    N, H, W, R, pooled, scale = 2, 30, 44, 40, (7, 7), 0.25
    dy16 = rng.standard_normal((R, C) + pooled).astype(np.float16)
    c = np.stack([rng.uniform(0, W / scale, R), rng.uniform(0, H / scale, R)], 1)
    wh = np.stack([rng.uniform(2, W / scale, R), rng.uniform(2, H / scale, R)], 1)
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    want = oracle.backward(dy16.astype(np.float32), rois, (N, C, H, W), scale, S, impl='ordered')
    dx = abi.backward(abi.to_dev(dy16), abi.to_dev(rois), (N, C, H, W), scale, S, assign=True)
    assert dx.dtype == torch.float16
    assert_parity(dx.cpu().numpy().astype(np.float32), want.astype(np.float16).astype(np.float32), FP16_TOL, 'assign')
    base = rng.standard_normal((N, C, H, W)).astype(np.float16)
    dx = abi.backward(abi.to_dev(dy16), abi.to_dev(rois), (N, C, H, W), scale, S, dx=abi.to_dev(base))
    assert_parity(dx.cpu().numpy().astype(np.float32),
                  (want + base.astype(np.float32)).astype(np.float16).astype(np.float32), FP16_TOL, 'accumulate')


@pytest.mark.parametrize('quads', [1, 0])
@pytest.mark.parametrize('split', [1, 4])
@pytest.mark.parametrize('columns', [56, 28])
@pytest.mark.parametrize('cfg,down', [('cfg1', 8), ('cfg2', 16), ('cfg3', 32)])
def test_both_tile_widths_of_the_backward(cfg, down, columns, split, quads):
    """The backward chooses 28-column tiles for small maps and 56-column ones
    otherwise, on small maps lets four wavefronts share a tile row's work list,
    and writes rows of maps whose width is a multiple of four 16 bytes at a
    time; here each width, both sharings and both ways of writing are forced on
    every configuration."""
    abi.set_impl('tiled')
    native.set_option('roialign_tile_columns', columns)
    native.set_option('roialign_row_split', split)
    native.set_option('roialign_row_quads', quads)
    w = workloads.make_workload(cfg, scale_down=down)
    scale, S = w['spatial_scale'], w['sampling_ratio']
    rois, dy = abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    want = oracle.backward(w['dy'], w['rois'], w['data'].shape, scale, S, impl='ordered')
    assert_parity(abi.backward(dy, rois, w['data'].shape, scale, S, assign=True).cpu().numpy(), want, BWD_TOL,
                  'bwd assign')
    seed = torch.ones(w['data'].shape, device='cuda')
    assert_parity(abi.backward(dy, rois, w['data'].shape, scale, S, dx=seed).cpu().numpy(), want + 1, BWD_TOL,
                  'bwd accumulate')
    dy_cl = dy.permute(0, 2, 3, 1).contiguous()
    n, c, h, wd = w['data'].shape
    if native.roialign_channels_last_supported(True, 4, c, h, wd, w['pooled_size'], S, rois.shape[0]):
        got = abi.backward_nhwc(dy_cl, rois, (n, h, wd, c), scale, S, assign=True).permute(0, 3, 1, 2)
        assert_parity(got.cpu().numpy(), want, BWD_TOL, 'bwd channels-last')


@pytest.mark.parametrize('C', [1, 6, 35])
def test_four_column_write_out_with_odd_channel_counts(C):
    """Maps whose width is a multiple of four are written four columns at a time
    by the lanes of a channel quad: channel counts that end inside a quad, and
    a dx that starts at an odd element (which takes the other way out)."""
    abi.set_impl('tiled')
    rng = np.random.default_rng(C)
    N, H, W, PH, PW, scale, S, R = 2, 21, 60, 5, 7, 0.5, 2, 40
    x1 = rng.uniform(-10, W / scale, R); y1 = rng.uniform(-10, H / scale, R)
    rois = np.stack([rng.integers(0, N, R), x1, y1, x1 + rng.uniform(1, 90, R), y1 + rng.uniform(1, 40, R)],
                    1).astype(np.float32)
    dy = rng.standard_normal((R, C, PH, PW)).astype(np.float32)
    want = oracle.backward(dy, rois, (N, C, H, W), scale, S, impl='ordered')
    d_dy, d_rois = abi.to_dev(dy), abi.to_dev(rois)
    assert_parity(abi.backward(d_dy, d_rois, (N, C, H, W), scale, S, assign=True).cpu().numpy(), want, BWD_TOL,
                  'bwd assign')
    room = torch.full((N * C * H * W + 1,), 3.0, device='cuda')
    for shift in (0, 1):   # a dx at a multiple of 16 bytes, and one element further
        seed = room[shift:shift + N * C * H * W].view(N, C, H, W)
        seed.fill_(3.0)
        assert_parity(abi.backward(d_dy, d_rois, (N, C, H, W), scale, S, dx=seed).cpu().numpy(), want + 3, BWD_TOL,
                      'bwd accumulate, shift {}'.format(shift))


@pytest.mark.parametrize('S', [2, 3])
def test_more_boxes_in_one_tile_than_the_list_builder_keeps_on_chip(S):
    """The pre-pass keeps a tile's list of boxes in LDS up to 4096 entries and in memory
    beyond: 5000 boxes on a map of one tile (with S = 3: about two list items per box)."""
    abi.set_impl('tiled')
    rng = np.random.default_rng(90 + S)
    N, C, H, W, PH, PW, scale, R = 1, 8, 16, 48, 2, 3, 1.0, 5000
    x1 = rng.uniform(-2, W, R); y1 = rng.uniform(-2, H, R)
    rois = np.stack([np.zeros(R), x1, y1, x1 + rng.uniform(0.5, 30, R), y1 + rng.uniform(0.5, 12, R)],
                    1).astype(np.float32)
    dy = rng.standard_normal((R, C, PH, PW)).astype(np.float32)
    want = oracle.backward(dy, rois, (N, C, H, W), scale, S, impl='ordered')
    d_dy, d_rois = abi.to_dev(dy), abi.to_dev(rois)
    native.set_option('kernel_timing', 1)
    try:
        first = abi.backward(d_dy, d_rois, (N, C, H, W), scale, S, assign=True)
        assert _last_bracketed_kernel() == 'backward_blocked_kernel'
    finally:
        native.set_option('kernel_timing', 0)
    assert_parity(first.cpu().numpy(), want, BWD_TOL, 'bwd assign')
    assert torch.equal(first, abi.backward(d_dy, d_rois, (N, C, H, W), scale, S, assign=True))


def _last_bracketed_kernel():
    import ctypes
    lib = native.library()
    lib.mobula_hip_last_kernel_ms.restype = ctypes.c_double
    lib.mobula_hip_last_kernel_ms.argtypes = [ctypes.POINTER(ctypes.c_char_p)]
    name = ctypes.c_char_p()
    ms = lib.mobula_hip_last_kernel_ms(ctypes.byref(name))
    return name.value.decode() if ms >= 0 and name.value else None


@pytest.mark.parametrize('pooled,S', [((28, 28), 2), ((32, 20), 2), ((17, 32), 1), ((9, 30), 3), ((32, 32), 0),
                                      ((28, 28), 4)])
def test_tiled_backward_with_large_pooled_sizes(pooled, S):
    """Up to 64 sample rows and columns per ROI (32 x 32 bins of 2 x 2 points, mask heads pool 28 x 28)
    stay on the tile owners; every element against the oracle."""
    abi.set_impl('tiled')
    rng = np.random.default_rng(7000 + pooled[0] + S)
    N, C, H, W, R, scale = 2, 40, 40, 72, 24, 0.25
    x = rng.random((N, C, H, W), dtype=np.float32)
    dyh = rng.standard_normal((R, C) + pooled).astype(np.float32)
    c = np.stack([rng.uniform(0, W / scale, R), rng.uniform(0, H / scale, R)], 1)
    wh = np.exp(rng.uniform(np.log(4), np.log(1.2 * W / scale), (R, 2)))
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    native.set_option('kernel_timing', 1)
    try:
        dx = abi.backward(abi.to_dev(dyh), abi.to_dev(rois), x.shape, scale, S, assign=True)
        assert _last_bracketed_kernel() == 'backward_blocked_kernel'
    finally:
        native.set_option('kernel_timing', 0)
    want = oracle.backward(dyh, rois, x.shape, scale, S, impl='ordered')
    assert_parity(dx.cpu().numpy(), want, BWD_TOL, 'bwd {} S={}'.format(pooled, S))
    y = abi.forward(abi.to_dev(x), abi.to_dev(rois), pooled, scale, S).cpu().numpy()
    assert_parity(y, oracle.forward(x, rois, pooled, scale, S), FWD_TOL, 'fwd {} S={}'.format(pooled, S))


def test_tiled_backward_beyond_two_gib_of_blocked_gradient():
    """11500 ROIs x 256 channels x 14 x 14: the channel-blocked copy of dy holds 2.3 GB (every channel block
    a slab of its own, addressed with 32-bit offsets).  Checked against the straightforward kernel on the
    same inputs and by the adjoint identity with the forward."""
    g = torch.Generator(device='cuda').manual_seed(77)
    N, C, H, W, R, pooled, scale, S = 8, 256, 128, 128, 11500, (14, 14), 0.125, 2
    size = torch.exp(torch.rand(R, 2, device='cuda', generator=g) * np.log(16.0) + np.log(32.0))
    centre = torch.rand(R, 2, device='cuda', generator=g) * 1024.0
    rois = torch.cat([torch.randint(0, N, (R, 1), device='cuda', generator=g).float(), centre - size / 2,
                      centre + size / 2], 1).contiguous()
    dy = torch.randn((R, C) + pooled, device='cuda', generator=g)
    x = torch.rand((N, C, H, W), device='cuda', generator=g)
    abi.set_impl('tiled')
    native.set_option('kernel_timing', 1)
    try:
        dx = abi.backward(dy, rois, x.shape, scale, S, assign=True)
        assert _last_bracketed_kernel() == 'backward_blocked_kernel'
    finally:
        native.set_option('kernel_timing', 0)
    y = abi.forward(x, rois, pooled, scale, S)
    lhs = float((y.double() * dy.double()).sum())
    rhs = float((x.double() * dx.double()).sum())
    assert abs(lhs - rhs) <= 1e-6 * float((y.double().abs() * dy.double().abs()).sum())
    del y
    abi.set_impl('naive')
    dx_n = abi.backward(dy, rois, x.shape, scale, S)
    scale_ = float(dx_n.abs().max())
    assert float((dx - dx_n).abs().max()) <= BWD_TOL * scale_


@pytest.mark.parametrize('columns', [56, 28])
@pytest.mark.parametrize('S', [0, 3, 4, 5, 7, 65])
def test_tiled_backward_with_larger_sampling_grids(S, columns):
    """Sampling grids other than 1 or 2 points per bin are merged for the tiled
    backward: one weight per row and per column a bin touches, the columns in
    windows of seven cells (S = 0 gives every ROI its own grid; a fixed grid of
    65 points is beyond what is merged and takes the plain kernel).
    Boxes: tiny, ordinary, wider than the map, partly off the map."""
    abi.set_impl('tiled')
    native.set_option('roialign_tile_columns', columns)
    rng = np.random.default_rng(40 + S)
    N, C, H, W, PH, PW, scale = 2, 32, 37, 53, 7, 6, 0.25
    R = 96 if S < 65 else 6
    x1 = rng.uniform(-30, W / scale, R); y1 = rng.uniform(-30, H / scale, R)
    bw = rng.choice([0.5, 8, 40, 150, 400], R) * rng.uniform(0.5, 1.5, R)
    bh = rng.choice([0.5, 8, 40, 150, 400], R) * rng.uniform(0.5, 1.5, R)
    rois = np.stack([rng.integers(0, N, R), x1, y1, x1 + bw, y1 + bh], 1).astype(np.float32)
    dy = rng.standard_normal((R, C, PH, PW)).astype(np.float32)
    want = oracle.backward(dy, rois, (N, C, H, W), scale, S, impl='ordered')
    d_dy, d_rois = abi.to_dev(dy), abi.to_dev(rois)
    first = abi.backward(d_dy, d_rois, (N, C, H, W), scale, S, assign=True)
    assert_parity(first.cpu().numpy(), want, BWD_TOL, 'bwd assign')
    if S < 65:   # (the plain kernel adds with atomics, in any order)
        again = abi.backward(d_dy, d_rois, (N, C, H, W), scale, S, assign=True)
        assert torch.equal(first, again), 'the tiled backward is deterministic'
    seed = torch.full((N, C, H, W), 2.0, device='cuda')
    assert_parity(abi.backward(d_dy, d_rois, (N, C, H, W), scale, S, dx=seed).cpu().numpy(), want + 2, BWD_TOL,
                  'bwd accumulate')
    if native.roialign_channels_last_supported(True, 4, C, H, W, (PH, PW), S, R):
        got = abi.backward_nhwc(d_dy.permute(0, 2, 3, 1).contiguous(), d_rois, (N, H, W, C), scale, S, assign=True)
        assert_parity(got.permute(0, 3, 1, 2).cpu().numpy(), want, BWD_TOL, 'bwd channels-last')


@pytest.mark.parametrize('impl', IMPLS)
@pytest.mark.parametrize('shape', [
    # N, C, H, W, R, pooled, scale, S
    (1, 1, 1, 1, 3, (1, 1), 1.0, 1),        # single-pixel map
    (2, 3, 5, 7, 11, (2, 3), 0.5, 0),       # tiny odd sizes, adaptive grid
    (3, 65, 33, 47, 37, (7, 7), 0.25, 2),   # channel count just over one block
    (2, 130, 18, 70, 50, (14, 14), 0.125, 2),
    (1, 7, 64, 64, 20, (5, 9), 0.3, 3),     # non-square pooling, S=3
    (2, 4, 40, 40, 25, (7, 7), 1.0, 5),     # dense grid
    (2, 36, 60, 90, 40, (7, 7), 0.25, 0),   # adaptive grid over the blocked layout, ragged last block
    (1, 8, 200, 160, 12, (3, 14), 1.0, 0),  # bins of up to 67 x 11 samples: several sample windows
    (2, 8, 50, 50, 30, (14, 7), 0.5, 4),    # more pooled rows than one set of row lists holds
])
def test_ragged_shapes(impl, shape):
    abi.set_impl(impl)
    N, C, H, W, R, pooled, scale, S = shape
    rng = np.random.default_rng(hash(shape) & 0xffff)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    ext_w, ext_h = W / scale, H / scale
    c = np.stack([rng.uniform(-0.2 * ext_w, 1.2 * ext_w, R), rng.uniform(-0.2 * ext_h, 1.2 * ext_h, R)], 1)
    wh = np.stack([rng.uniform(0, ext_w, R), rng.uniform(0, ext_h, R)], 1)
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    dy = rng.standard_normal((R, C) + pooled).astype(np.float32)
    y = abi.forward(abi.to_dev(x), abi.to_dev(rois), pooled, scale, S).cpu().numpy()
    assert_parity(y, oracle.forward(x, rois, pooled, scale, S), FWD_TOL, 'fwd')
    want = oracle.backward(dy, rois, x.shape, scale, S, impl='ordered')
    for assign in (False, True):
        dx = abi.backward(abi.to_dev(dy), abi.to_dev(rois), x.shape, scale, S, assign=assign)
        assert_parity(dx.cpu().numpy(), want, BWD_TOL, 'bwd assign=%s' % assign)


def test_random_shapes_both_layouts():
    # sixty seeded problems -- odd map sizes, boxes across the borders, tiny and empty boxes, image
    # numbers outside the batch, every kind of sampling grid, fp16 maps, both tile widths, split rows
    # and both write-outs of the backward -- against the oracle, in both layouts where channels-last
    # takes the shape
    abi.set_impl('auto')
    for case in range(60):
        rng = np.random.default_rng(31000 + case)
        N, C = int(rng.integers(1, 4)), int(rng.choice([4, 8, 12, 32, 36, 64, 68, 100]))
        H, W, R = int(rng.integers(1, 70)), int(rng.integers(1, 130)), int(rng.integers(0, 60))
        if rng.integers(0, 2):
            W = (W + 3) // 4 * 4
        PH, PW = int(rng.integers(1, 15)), int(rng.integers(1, 20))
        S = int(rng.choice([0, 0, 1, 2, 2, 3, 4, 5, 7]))
        scale = float(rng.choice([1.0, 0.5, 0.25, 0.125, 0.3]))
        fp16 = bool(rng.integers(0, 4) == 0)
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        ew, eh = W / scale, H / scale
        kind = rng.integers(0, 4, R)
        c = np.stack([rng.uniform(-0.3 * ew, 1.3 * ew, R), rng.uniform(-0.3 * eh, 1.3 * eh, R)], 1)
        wh = np.stack([rng.uniform(0, ew, R), rng.uniform(0, eh, R)], 1)
        wh[kind == 1] *= 0.05
        wh[kind == 2] = 0.0
        rois = np.concatenate([rng.integers(-1, N + 1, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
        dy = rng.standard_normal((R, C, PH, PW)).astype(np.float32)
        native.set_option('roialign_tile_columns', int(rng.choice([0, 28, 56])))
        native.set_option('roialign_row_split', int(rng.choice([0, 1, 4])))
        native.set_option('roialign_row_quads', int(rng.integers(0, 2)))
        what = 'case {}: N{} C{} {}x{} R{} pooled {}x{} S{} scale {} fp16 {}'.format(case, N, C, H, W, R, PH, PW, S,
                                                                                   scale, fp16)
        print(what, flush=True)
        # (the oracle indexes the map with the box's image number: boxes that name no image are
        # left out for it; the library gives them zeros)
        ok = (rois[:, 0] >= 0) & (rois[:, 0] < N)
        x_in = x.astype(np.float16) if fp16 else x
        want = oracle.forward(x_in.astype(np.float32), rois[ok], (PH, PW), scale, S)
        if fp16:
            want = want.astype(np.float16).astype(np.float32)
        tol = FP16_TOL if fp16 else FWD_TOL
        y = abi.forward(abi.to_dev(x_in), abi.to_dev(rois), (PH, PW), scale, S).cpu().numpy().astype(np.float32)
        if ok.any():
            assert_parity(y[ok], want, tol, what + ' fwd')
        assert np.abs(y[~ok]).sum() == 0, what
        if C % (8 if fp16 else 4) == 0:
            y_l = abi.forward_nhwc(abi.to_dev(x_in.transpose(0, 2, 3, 1)), abi.to_dev(rois), (PH, PW), scale, S)
            y_l = y_l.cpu().numpy().astype(np.float32).transpose(0, 3, 1, 2)
            if ok.any():
                assert_parity(y_l[ok], want, tol, what + ' fwd channels-last')
        if fp16:
            continue
        want_dx = oracle.backward(dy[ok], rois[ok], x.shape, scale, S, impl='ordered') if ok.any() else np.zeros_like(x)
        dx = abi.backward(abi.to_dev(dy), abi.to_dev(rois), x.shape, scale, S, assign=bool(case % 2)).cpu().numpy()
        assert_parity(dx, want_dx, BWD_TOL, what + ' bwd')
        if native.roialign_channels_last_supported(True, 4, C, H, W, (PH, PW), S, R):
            dx_l = abi.backward_nhwc(abi.to_dev(dy.transpose(0, 2, 3, 1)), abi.to_dev(rois), (N, H, W, C), scale, S,
                                     assign=bool(case % 2))
            assert_parity(dx_l.cpu().numpy().transpose(0, 3, 1, 2), want_dx, BWD_TOL, what + ' bwd channels-last')


@pytest.mark.parametrize('pooled', [(3, 60), (2, 68), (1, 69), (40, 9)])
@pytest.mark.parametrize('S', [2, 0])
def test_forward_with_very_wide_or_tall_pooled_maps(pooled, S):
    # up to 68 pooled columns go through the staged gather (one pooled row per pass at that
    # width), 69 through the straightforward kernel; 40 pooled rows of 2 samples are more row
    # samples than the gather holds at a time
    abi.set_impl('auto')
    N, C, H, W, R, scale = 2, 36, 50, 90, 14, 0.5
    rng = np.random.default_rng(99 + pooled[1] + S)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    ext_w, ext_h = W / scale, H / scale
    c = np.stack([rng.uniform(0, ext_w, R), rng.uniform(0, ext_h, R)], 1)
    wh = np.stack([rng.uniform(0, ext_w, R), rng.uniform(0, ext_h, R)], 1)
    wh[::5] *= 0.05
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    y = abi.forward(abi.to_dev(x), abi.to_dev(rois), pooled, scale, S).cpu().numpy()
    assert_parity(y, oracle.forward(x, rois, pooled, scale, S), FWD_TOL, 'fwd')
    dy = rng.standard_normal((R, C) + pooled).astype(np.float32)
    dx = abi.backward(abi.to_dev(dy), abi.to_dev(rois), x.shape, scale, S, assign=True).cpu().numpy()
    assert_parity(dx, oracle.backward(dy, rois, x.shape, scale, S, impl='ordered'), BWD_TOL, 'bwd')


@pytest.mark.parametrize('layout', ['nchw', 'nhwc'])
@pytest.mark.parametrize('pooled,S', [((7, 7), 2), ((14, 14), 2), ((5, 9), 1), ((16, 3), 2)])
def test_boxes_whose_samples_share_rows_and_columns(pooled, S, layout):
    # Boxes of 0 .. 1.5 pooled sizes in pixels: samples less than a pixel apart, so a map row (or
    # column) serves several samples of a bin and of neighbouring bins -- the forward gather fetches
    # it once and carries its column sum along, the list builder folds a bin's two taps on it into
    # one.  Boxes sit anywhere, also across the map's borders, where the two rows (columns) of
    # a sample collapse into one.
    abi.set_impl('auto')
    N, C, H, W, R, scale = 2, 40, 23, 37, 120, 0.5
    rng = np.random.default_rng(4242 + 7 * pooled[0] + S)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    ext_w, ext_h = W / scale, H / scale
    c = np.stack([rng.uniform(-3, ext_w + 3, R), rng.uniform(-3, ext_h + 3, R)], 1)
    wh = np.stack([rng.uniform(0, 1.5 * pooled[1] / scale, R), rng.uniform(0, 1.5 * pooled[0] / scale, R)], 1)
    wh[::7] = 0.0                                        # boxes without an extent
    c[1::9, 1] = ext_h - rng.uniform(0, 1.0, len(c[1::9]))   # on the last row
    c[2::11, 0] = rng.uniform(-1.0, 0.5, len(c[2::11]))      # on the first column
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    dy = rng.standard_normal((R, C) + pooled).astype(np.float32)
    want_y = oracle.forward(x, rois, pooled, scale, S)
    want_dx = oracle.backward(dy, rois, x.shape, scale, S, impl='ordered')
    if layout == 'nchw':
        y = abi.forward(abi.to_dev(x), abi.to_dev(rois), pooled, scale, S).cpu().numpy()
        dx = abi.backward(abi.to_dev(dy), abi.to_dev(rois), x.shape, scale, S, assign=True).cpu().numpy()
    else:
        y = abi.forward_nhwc(abi.to_dev(x.transpose(0, 2, 3, 1)), abi.to_dev(rois), pooled, scale, S)
        y = y.cpu().numpy().transpose(0, 3, 1, 2)
        dx = abi.backward_nhwc(abi.to_dev(dy.transpose(0, 2, 3, 1)), abi.to_dev(rois), (N, H, W, C), scale, S,
                               assign=True).cpu().numpy().transpose(0, 3, 1, 2)
    assert_parity(y, want_y, FWD_TOL, 'fwd')
    assert_parity(dx, want_dx, BWD_TOL, 'bwd')
    # 16-bit maps take the path that shares rows within a bin only
    x16 = x.astype(np.float16)
    if layout == 'nchw':
        y16 = abi.forward(abi.to_dev(x16), abi.to_dev(rois), pooled, scale, S).cpu().numpy()
    else:
        y16 = abi.forward_nhwc(abi.to_dev(np.ascontiguousarray(x16.transpose(0, 2, 3, 1))), abi.to_dev(rois), pooled,
                               scale, S).cpu().numpy().transpose(0, 3, 1, 2)
    want16 = oracle.forward(x16.astype(np.float32), rois, pooled, scale, S)
    assert_parity(y16.astype(np.float32), want16.astype(np.float16).astype(np.float32), FP16_TOL, 'fwd fp16')


@pytest.mark.parametrize('shape', [
    # N, C, H, W, R, pooled, scale, S
    (3, 68, 33, 47, 37, (7, 7), 0.25, 2),     # ragged last channel block
    (2, 128, 18, 70, 50, (14, 14), 0.125, 2),
    (2, 32, 40, 40, 25, (7, 7), 1.0, 1),
])
def test_channels_last_entry_points(shape):
    # map [N,H,W,C], pooled tensor [R,PH,PW,C]: same numbers as the NCHW oracle, transposed
    abi.set_impl('auto')
    N, C, H, W, R, pooled, scale, S = shape
    rng = np.random.default_rng(hash(shape) & 0xffff)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    ext_w, ext_h = W / scale, H / scale
    c = np.stack([rng.uniform(-0.2 * ext_w, 1.2 * ext_w, R), rng.uniform(-0.2 * ext_h, 1.2 * ext_h, R)], 1)
    wh = np.stack([rng.uniform(0, ext_w, R), rng.uniform(0, ext_h, R)], 1)
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    dy = rng.standard_normal((R, C) + pooled).astype(np.float32)
    y = abi.forward_nhwc(abi.to_dev(x.transpose(0, 2, 3, 1)), abi.to_dev(rois), pooled, scale, S)
    assert_parity(y.cpu().numpy().transpose(0, 3, 1, 2), oracle.forward(x, rois, pooled, scale, S), FWD_TOL, 'fwd')
    want = oracle.backward(dy, rois, x.shape, scale, S, impl='ordered')
    dy_l = abi.to_dev(dy.transpose(0, 2, 3, 1))
    for assign in (False, True):
        dx = abi.backward_nhwc(dy_l, abi.to_dev(rois), (N, H, W, C), scale, S, assign=assign)
        assert_parity(dx.cpu().numpy().transpose(0, 3, 1, 2), want, BWD_TOL, 'bwd assign=%s' % assign)
    # accumulation into an existing gradient
    base = rng.standard_normal((N, H, W, C)).astype(np.float32)
    dx = abi.backward_nhwc(dy_l, abi.to_dev(rois), (N, H, W, C), scale, S, dx=abi.to_dev(base))
    assert_parity(dx.cpu().numpy().transpose(0, 3, 1, 2), want + base.transpose(0, 3, 1, 2), BWD_TOL, 'accumulate')


def test_channels_last_fp16_and_adaptive_grid():
    abi.set_impl('auto')
    rng = np.random.default_rng(77)
    N, C, H, W, R, pooled, scale = 2, 72, 30, 44, 60, (7, 7), 0.25
    x16 = rng.standard_normal((N, C, H, W)).astype(np.float16)
    c = np.stack([rng.uniform(0, W / scale, R), rng.uniform(0, H / scale, R)], 1)
    wh = np.stack([rng.uniform(2, W / scale, R), rng.uniform(2, H / scale, R)], 1)
    rois = np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32)
    for S in (2, 0):
        y = abi.forward_nhwc(abi.to_dev(x16.transpose(0, 2, 3, 1)), abi.to_dev(rois), pooled, scale, S)
        want = oracle.forward(x16.astype(np.float32), rois, pooled, scale, S)
        assert_parity(y.cpu().numpy().astype(np.float32).transpose(0, 3, 1, 2),
                      want.astype(np.float16).astype(np.float32), FP16_TOL, 'fp16 S=%d' % S)


def test_channels_last_rejects_what_it_does_not_take():
    x = torch.zeros(1, 8, 8, 6, device='cuda')          # six channels: no multiple of four
    rois = torch.tensor([[0, 1, 1, 6, 6]], device='cuda', dtype=torch.float32)
    with pytest.raises(RuntimeError, match='channels-last'):
        abi.forward_nhwc(x, rois, (2, 2), 1.0, 2)
    dy = torch.zeros(1, 7, 33, 8, device='cuda')         # 33 pooled columns: more than the backward's lists hold
    with pytest.raises(RuntimeError, match='channels-last'):
        abi.backward_nhwc(dy, rois, (1, 8, 8, 8), 1.0, 2)
    dy = torch.zeros(1, 2, 2, 8, device='cuda')          # a fixed grid of more than 64 points per bin and axis
    assert not native.roialign_channels_last_supported(True, 4, 8, 8, 8, (2, 2), 65, 1)
    with pytest.raises(RuntimeError, match='channels-last'):
        abi.backward_nhwc(dy, rois, (1, 8, 8, 8), 1.0, 65)
    # an adaptive grid is taken (its bins' weights are merged)
    assert native.roialign_channels_last_supported(True, 4, 8, 8, 8, (2, 2), 0, 1)
    assert abi.backward_nhwc(dy, rois, (1, 8, 8, 8), 1.0, 0, assign=True).abs().sum().item() == 0.0
    # the library is usable afterwards
    assert abi.forward_nhwc(torch.zeros(1, 8, 8, 8, device='cuda'), rois, (2, 2), 1.0, 2).shape == (1, 2, 2, 8)


def test_a_backward_with_a_dense_grid_can_be_recorded_too():
    """The merged lists of a dense sampling grid are sized by a number that comes back from
    the device, which a capturing stream cannot wait for: such a call is recorded with the
    straightforward kernel (atomic adds: same sums, any order) and the replays give the
    direct call's result within the tolerance."""
    rng = np.random.default_rng(123)
    N, C, H, W, R, pooled, scale, S = 2, 16, 40, 60, 50, (5, 6), 0.5, 3
    ext = np.array([W / scale, H / scale])
    c = rng.uniform(0, 1, (R, 2)) * ext
    wh = rng.uniform(2, 60, (R, 2))
    rois = abi.to_dev(np.concatenate([rng.integers(0, N, (R, 1)), c - wh / 2, c + wh / 2], 1).astype(np.float32))
    dy = abi.to_dev(rng.standard_normal((R, C) + pooled).astype(np.float32))
    dx = torch.empty((N, C, H, W), device='cuda')
    want = abi.backward(dy, rois, dx.shape, scale, S, assign=True).clone()   # the tile owners
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        abi.backward(dy, rois, dx.shape, scale, S, dx=dx, assign=True, stream=torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        dx.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_parity(dx.cpu().numpy(), want.cpu().numpy(), BWD_TOL, 'replay %d' % replay)
    native.unpin_workspace()


F64_TOL = 1e-12   # binary64: only the backward's summation order may differ


@pytest.mark.parametrize('S', [2, 0])
def test_double_instantiation(S):
    """roi_align_forward_6b9e6c9b (the reference's <double> forward) and the two
    double backward entry points, against the double oracle and the fixtures the
    compiled reference wrote."""
    folder = os.path.join(GOLDEN, 'f64')
    for name in sorted(f for f in os.listdir(folder) if f.endswith('.npz')):
        z = np.load(os.path.join(folder, name))
        pooled = tuple(int(v) for v in z['pooled_size'])
        y = abi.forward(abi.to_dev(z['data']), abi.to_dev(z['rois']), pooled, float(z['spatial_scale']),
                        int(z['sampling_ratio']))
        assert y.dtype == torch.float64
        np.testing.assert_array_equal(y.cpu().numpy(), z['y'], err_msg=name)   # same operations, same order
    rng = np.random.default_rng(77 + S)
    N, C, H, W, R, pooled, scale = 3, 5, 21, 30, 50, (5, 6), 0.3
    xh = rng.standard_normal((N, C, H, W))
    c, wh = rng.uniform(-10, 110, size=(R, 2)), rng.uniform(0, 90, size=(R, 2))
    rh = np.concatenate([rng.integers(0, N, size=(R, 1)), c - wh / 2, c + wh / 2], axis=1)
    rh[0, 1:] = [400, 400, 500, 500]
    rh[1, 1:] = [20, 20, 20, 20]
    dyh = rng.standard_normal((R, C) + pooled)
    x, rois, dy = abi.to_dev(xh), abi.to_dev(rh), abi.to_dev(dyh)
    np.testing.assert_array_equal(abi.forward(x, rois, pooled, scale, S).cpu().numpy(),
                                  oracle.forward_f64(xh, rh, pooled, scale, S))
    want_dx = oracle.backward_f64(dyh, rh, xh.shape, scale, S)
    assert_parity(abi.backward(dy, rois, x.shape, scale, S).cpu().numpy(), want_dx, F64_TOL, 'bwd')
    assert_parity(abi.backward(dy, rois, x.shape, scale, S, assign=True).cpu().numpy(), want_dx, F64_TOL,
                  'bwd assign')
    seed = torch.ones_like(x)
    assert_parity(abi.backward(dy, rois, x.shape, scale, S, dx=seed).cpu().numpy(), want_dx + 1.0, F64_TOL,
                  'bwd accumulate')
    # without declared extents the image count comes from the (double) boxes
    np.testing.assert_array_equal(abi.forward(x, rois, pooled, scale, S, declare_extents=False).cpu().numpy(),
                                  oracle.forward_f64(xh, rh, pooled, scale, S))


def test_asynchronous_calls_on_two_streams_and_two_threads():
    """The library's scratch memory (the blocked copy of the map, the backward's
    lists) belongs to the calling thread: a thread that moves to another stream is
    ordered behind its own previous call, and two threads never share a buffer."""
    import threading
    cases = []
    for k, (cfg, down) in enumerate([('cfg2', 16), ('cfg1', 8)]):
        w = workloads.make_workload(cfg, scale_down=down)
        want = oracle.forward(w['data'], w['rois'], w['pooled_size'], w['spatial_scale'], w['sampling_ratio'])
        want_dx = oracle.backward(w['dy'], w['rois'], w['data'].shape, w['spatial_scale'],
                                  w['sampling_ratio'], impl='ordered')
        cases.append((w, abi.to_dev(w['data']), abi.to_dev(w['rois']), abi.to_dev(w['dy']), want, want_dx))
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()

    def run(order, out):
        for k in order:   # back to back, nothing waits in between
            w, x, rois, dy, _, _ = cases[k]
            s = streams[k].cuda_stream
            y = abi.forward(x, rois, w['pooled_size'], w['spatial_scale'], w['sampling_ratio'], stream=s)
            dx = abi.backward(dy, rois, x.shape, w['spatial_scale'], w['sampling_ratio'], assign=True, stream=s)
            out.append((k, y, dx))

    # one thread, alternating streams
    got = []
    run([0, 1, 0, 1, 1, 0], got)
    torch.cuda.synchronize()
    # two threads at once, one stream each
    per_thread = [[], []]
    threads = [threading.Thread(target=run, args=([k] * 4, per_thread[k])) for k in (0, 1)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    for k, y, dx in got + per_thread[0] + per_thread[1]:
        assert_parity(y.cpu().numpy(), cases[k][4], FWD_TOL, 'fwd')
        assert_parity(dx.cpu().numpy(), cases[k][5], BWD_TOL, 'bwd')


@pytest.mark.parametrize('layout', ['nchw', 'nhwc'])
def test_calls_recorded_in_a_graph_replay_bit_for_bit(layout):
    """After one ordinary call (which sizes the workspace) a forward and a
    backward on a capturing stream are recorded, not run; every replay, with
    ordinary calls and synchronisations in between, gives the bits of a direct
    call.  (The backward forks to a second stream and joins it inside the call.)"""
    w = workloads.make_workload('cfg2')   # full size: dy is large enough for the backward to fork
    scale, S, pooled = w['spatial_scale'], w['sampling_ratio'], w['pooled_size']
    nhwc = layout == 'nhwc'
    x = abi.to_dev(w['data'].transpose(0, 2, 3, 1) if nhwc else w['data'])
    dy = abi.to_dev(w['dy'].transpose(0, 2, 3, 1) if nhwc else w['dy'])
    rois = abi.to_dev(w['rois'])
    fwd, bwd = (abi.forward_nhwc, abi.backward_nhwc) if nhwc else (abi.forward, abi.backward)
    dx = torch.empty_like(x)
    stream = torch.cuda.Stream()

    def direct():
        with torch.cuda.stream(stream):
            y = fwd(x, rois, pooled, scale, S, stream=stream.cuda_stream)
            bwd(dy, rois, x.shape, scale, S, dx=dx, assign=True, stream=stream.cuda_stream)
        stream.synchronize()
        return y.clone(), dx.clone()

    torch.cuda.synchronize()
    native.release_workspace()   # (earlier tests may have left a larger one: this test wants it sized by its own calls)
    y_want, dx_want = direct()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        inner = torch.cuda.current_stream().cuda_stream
        y_graph = fwd(x, rois, pooled, scale, S, stream=inner)
        bwd(dy, rois, x.shape, scale, S, dx=dx, assign=True, stream=inner)
    for replay in range(4):
        dx.fill_(7.0); y_graph.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y_want), 'forward, replay %d' % replay
        assert torch.equal(dx, dx_want), 'backward, replay %d' % replay
        y_now, dx_now = direct()            # ordinary calls between the replays
        assert torch.equal(y_now, y_want) and torch.equal(dx_now, dx_want)
    # the graph refers to the workspace by address: while it may be replayed the buffer is
    # neither given back nor replaced by a larger one (host-side book-keeping, nothing faults)
    held = native.workspace_bytes()
    with pytest.raises(RuntimeError, match='recorded graph'):
        native.release_workspace()
    big = torch.zeros((8, 256, 200, 336), device='cuda')
    if nhwc:
        big = big.permute(0, 2, 3, 1).contiguous()
    dy_big = torch.zeros_like(abi.to_dev(w['dy'].transpose(0, 2, 3, 1) if nhwc else w['dy'])).repeat(3, 1, 1, 1)
    rois_big = rois.repeat(3, 1)
    with pytest.raises(RuntimeError, match='recorded graph'):
        bwd(dy_big, rois_big, big.shape, scale, S, assign=True)
    assert native.workspace_bytes() == held
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(dx, dx_want)
    del graph
    native.unpin_workspace()
    assert bwd(dy_big, rois_big, big.shape, scale, S, assign=True).shape == big.shape
    assert native.workspace_bytes() > held


@pytest.mark.parametrize('impl', IMPLS)
def test_non_finite_gradient_of_one_roi_stays_in_its_cells(impl):
    """dy of ROI 0 is infinite; ROI 1 lies in the same tile rows but touches
    other cells: its part of dx is what it would be without ROI 0."""
    abi.set_impl(impl)
    rng = np.random.default_rng(5)
    N, C, H, W, pooled, scale, S = 1, 8, 16, 56, (3, 3), 1.0, 2
    rois = np.array([[0, 1.3, 2.2, 9.1, 12.7], [0, 30.4, 1.5, 41.2, 13.3]], np.float32)
    dy = rng.standard_normal((2, C) + pooled).astype(np.float32)
    alone = dy.copy(); alone[0] = 0.0
    want = oracle.backward(alone, rois, (N, C, H, W), scale, S, impl='ordered')
    dy[0] = np.inf
    for S_ in (S, 0, 3):
        want = oracle.backward(alone, rois, (N, C, H, W), scale, S_, impl='ordered')
        got = abi.backward(abi.to_dev(dy), abi.to_dev(rois), (N, C, H, W), scale, S_, assign=True).cpu().numpy()
        assert np.isfinite(got[..., 28:]).all(), 'S=%d' % S_
        assert_parity(got[..., 28:], want[..., 28:], BWD_TOL, 'cells of ROI 1, S=%d' % S_)
        assert not np.isfinite(got[..., :12]).all()


def test_workspace_can_be_given_back():
    """The scratch buffer grows with the largest call of the thread; a caller
    may release it between phases, and the next call allocates afresh."""
    w = workloads.make_workload('cfg1', scale_down=4)
    scale, S, pooled = w['spatial_scale'], w['sampling_ratio'], w['pooled_size']
    x, rois, dy = abi.to_dev(w['data']), abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    abi.set_impl('tiled')
    y = abi.forward(x, rois, pooled, scale, S)
    dx = abi.backward(dy, rois, x.shape, scale, S, assign=True)
    held = native.workspace_bytes()
    assert held > 0
    assert native.release_workspace() == held
    assert native.workspace_bytes() == 0 and native.release_workspace() == 0
    assert torch.equal(abi.forward(x, rois, pooled, scale, S), y)
    assert torch.equal(abi.backward(dy, rois, x.shape, scale, S, assign=True), dx)
    assert native.workspace_bytes() > 0


@pytest.mark.parametrize('impl', IMPLS)
def test_empty_roi_list_and_out_of_range_batch(impl):
    abi.set_impl(impl)
    x = torch.rand(2, 4, 8, 8, device='cuda')
    none = torch.zeros(0, 5, device='cuda')
    assert abi.forward(x, none, (7, 7), 1.0, 2).shape == (0, 4, 7, 7)
    dy0 = torch.zeros(0, 4, 7, 7, device='cuda')
    assert float(abi.backward(dy0, none, x.shape, 1.0, 2, assign=True).abs().sum()) == 0
    # a batch index beyond the map reads nothing and scatters nothing
    rois = torch.tensor([[0, 1, 1, 6, 6], [5, 1, 1, 6, 6], [-3, 1, 1, 6, 6]], device='cuda',
                        dtype=torch.float32)
    y = abi.forward(x, rois, (2, 2), 1.0, 2)
    assert float(y[1:].abs().sum()) == 0 and float(y[0].abs().sum()) > 0
    dy = torch.ones(3, 4, 2, 2, device='cuda')
    dx = abi.backward(dy, rois, x.shape, 1.0, 2, assign=True)
    assert abs(float(dx.sum()) - 16.0) < 1e-4 and float(dx[1].abs().sum()) == 0


@pytest.mark.parametrize('impl', IMPLS)
def test_boxes_far_larger_than_the_map(impl):
    """An adaptive grid has ceil(box / pooled) points per bin and axis: 1143 here, of which
    a dozen fall on the map.  The kernels visit only the samples that can be valid (found
    by bisection with the reference's own coordinate formula), so the results must still be
    the reference's."""
    abi.set_impl(impl)
    rng = np.random.default_rng(21)
    xh = rng.standard_normal((2, 8, 12, 16)).astype(np.float32)
    rh = np.array([[0, -3000, -2000, 5000, 4000], [1, -500, 3, 40, 9], [0, 2, -900, 11, 700],
                   [1, 1, 1, 14, 10]], dtype=np.float32)
    pooled = (3, 2)
    x, rois = abi.to_dev(xh), abi.to_dev(rh)
    y = abi.forward(x, rois, pooled, 1.0, 0).cpu().numpy()
    assert_parity(y, oracle.forward(xh, rh, pooled, 1.0, 0), FWD_TOL, 'fwd')
    dyh = rng.standard_normal(y.shape).astype(np.float32)
    dx = abi.backward(abi.to_dev(dyh), rois, x.shape, 1.0, 0, assign=True).cpu().numpy()
    assert_parity(dx, oracle.backward(dyh, rh, xh.shape, 1.0, 0, impl='ordered'), BWD_TOL, 'bwd')
    x64, r64 = abi.to_dev(xh.astype(np.float64)), abi.to_dev(rh.astype(np.float64))
    np.testing.assert_array_equal(abi.forward(x64, r64, pooled, 1.0, 0).cpu().numpy(),
                                  oracle.forward_f64(xh, rh, pooled, 1.0, 0))


@pytest.mark.parametrize('impl', IMPLS)
def test_non_finite_boxes_end_and_stay_inside_the_map(impl):
    """Boxes with infinite or NaN corners: the kernels must return (an infinite box has an
    adaptive grid of 2^31 points per bin) and must not leave their buffers.  A box whose
    samples are all outside gives zeros; coordinates that are not numbers give NaN in that
    box's own outputs and, in the backward, in its own image.  Such boxes sit on image 1
    here; image 0 must come out as if they were not there."""
    abi.set_impl(impl)
    rng = np.random.default_rng(11)
    xh = rng.standard_normal((2, 8, 20, 24)).astype(np.float32)
    inf, nan = np.inf, np.nan
    rh = np.array([[0, 4, 4, 60, 50],          # ordinary
                   [0, 5, inf, 9, inf],        # below the map: no valid sample
                   [inf, 1, 1, 9, 9],          # no such image
                   [0, 10, 12, 44, 70],        # ordinary
                   [nan, 1, 1, 9, 9],          # batch index NaN: becomes image 0 on the GPU, an ordinary box
                   [1, -inf, 3, 20, 30], [1, 2, 2, inf, 40], [1, nan, 3, 20, 30], [1, 3, 3, nan, nan],
                   [1, -inf, -inf, inf, inf]], dtype=np.float32)
    ordinary = [0, 3]
    x, rois = abi.to_dev(xh), abi.to_dev(rh)
    as_zero_batch = rh[[0, 3, 4]].copy()
    as_zero_batch[:, 0] = 0
    for S in (2, 0):
        y = abi.forward(x, rois, (7, 7), 0.25, S).cpu().numpy()
        assert_parity(y[ordinary], oracle.forward(xh, rh[ordinary], (7, 7), 0.25, S), FWD_TOL, 'ordinary boxes')
        assert np.abs(y[[1, 2]]).max() == 0
        dyh = rng.standard_normal(y.shape).astype(np.float32)
        dx = abi.backward(abi.to_dev(dyh), rois, x.shape, 0.25, S, assign=True).cpu().numpy()
        want = oracle.backward(dyh[[0, 3, 4]], as_zero_batch, x.shape, 0.25, S, impl='ordered')
        assert_parity(dx[0], want[0], BWD_TOL, 'image 0')


@pytest.mark.parametrize('impl', IMPLS)
def test_without_declared_extents(impl):
    # plain C callers do not say how many images there are: N comes from the rois
    abi.set_impl(impl)
    w = workloads.make_workload('cfg1', scale_down=32)
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    x, rois, dy = abi.to_dev(w['data']), abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    y = abi.forward(x, rois, pooled, scale, S, declare_extents=False).cpu().numpy()
    assert_parity(y, oracle.forward(w['data'], w['rois'], pooled, scale, S), FWD_TOL, 'fwd')
    dx = abi.backward(dy, rois, x.shape, scale, S, declare_extents=False).cpu().numpy()
    assert_parity(dx, oracle.backward(w['dy'], w['rois'], x.shape, scale, S, impl='ordered'),
                  BWD_TOL, 'bwd')


def test_shape_errors_are_reported_not_fatal():
    x = torch.rand(2, 4, 8, 8, device='cuda')
    rois = torch.zeros(3, 5, device='cuda')
    with pytest.raises(RuntimeError, match='rois holds'):
        _bad_rois_call(x)
    # the library is still usable afterwards
    assert abi.forward(x, rois, (2, 2), 1.0, 2).shape == (3, 4, 2, 2)


def test_an_error_belongs_to_the_call_that_caused_it():
    # a caller of the reference ABI (void functions) that never asks for the error text:
    # the call after a failed one computes
    import ctypes
    lib = native.library()
    x = torch.rand(2, 4, 8, 8, device='cuda')
    rois = torch.tensor([[0, 1, 1, 6, 6], [1, 0, 2, 5, 7], [1, 2, 2, 4, 4]], dtype=torch.float32, device='cuda')
    want = abi.forward(x, rois, (2, 2), 1.0, 2)
    bad_rois = torch.zeros(2, 5, device='cuda')
    y = torch.full((3, 4, 2, 2), float('nan'), device='cuda')
    abi._begin([-1, x.numel(), -1, -1, -1, -1, -1, -1, -1, bad_rois.numel(), y.numel()])
    lib.roi_align_forward_ab78de3c(ctypes.c_int(0), ctypes.c_int(y.numel()), abi._ptr(x),
                                   *abi._geom(1.0, 4, 8, 8, 2, 2, 2), abi._ptr(bad_rois), abi._ptr(y))
    assert lib.mobula_hip_last_error()          # reported ...
    assert torch.isnan(y).all()                 # ... and nothing computed
    # no mobula_hip_clear_error() here
    abi._begin([-1, x.numel(), -1, -1, -1, -1, -1, -1, -1, rois.numel(), y.numel()])
    lib.roi_align_forward_ab78de3c(ctypes.c_int(0), ctypes.c_int(y.numel()), abi._ptr(x),
                                   *abi._geom(1.0, 4, 8, 8, 2, 2, 2), abi._ptr(rois), abi._ptr(y))
    assert not lib.mobula_hip_last_error()
    assert torch.equal(y, want)
    # the same for a bad num_images of the overwriting backward, and a channels-last call with host memory
    dx = torch.full((2, 4, 8, 8), float('nan'), device='cuda')
    dy = torch.rand(3, 4, 2, 2, device='cuda')
    lib.roi_align_backward_assign_a8793cbe(ctypes.c_int(0), ctypes.c_int(dy.numel()), abi._ptr(dy),
                                           *abi._geom(1.0, 4, 8, 8, 2, 2, 2), ctypes.c_int(-1), abi._ptr(dx),
                                           abi._ptr(rois))
    assert lib.mobula_hip_last_error()
    got = abi.backward(dy, rois, (2, 4, 8, 8), 1.0, 2, assign=True)
    assert torch.isfinite(got).all() and float(got.abs().sum()) > 0


def _bad_rois_call(x):
    import ctypes
    from mobulaop_amd import native
    lib = native.library()
    rois = torch.zeros(2, 5, device='cuda')
    y = torch.empty(3, 4, 2, 2, device='cuda')
    ext = [-1, x.numel(), -1, -1, -1, -1, -1, -1, -1, rois.numel(), y.numel()]
    abi._begin(ext)
    lib.roi_align_forward_ab78de3c(ctypes.c_int(0), ctypes.c_int(y.numel()), abi._ptr(x),
                                   *abi._geom(1.0, 4, 8, 8, 2, 2, 2), abi._ptr(rois), abi._ptr(y))
    abi._end(lib)


# ---------------------------------------------------------------------------
# Full benchmark sizes: size-independent properties + oracle on a ROI subset.
# ---------------------------------------------------------------------------
@pytest.mark.parametrize('cfg', ['cfg2', 'cfg3'])
def test_full_size_properties(cfg):
    w = workloads.make_workload(cfg)
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    x, rois, dy = abi.to_dev(w['data']), abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    abi.set_impl('auto')
    y = abi.forward(x, rois, pooled, scale, S)
    dx = abi.backward(dy, rois, x.shape, scale, S, assign=True)
    # (1) oracle on a subset of the ROIs (forward rows are independent)
    pick = np.random.default_rng(0).choice(w['rois'].shape[0], 48, replace=False)
    want = oracle.forward(w['data'], w['rois'][pick], pooled, scale, S)
    assert_parity(y[torch.from_numpy(pick).cuda()].cpu().numpy(), want, FWD_TOL, cfg + ' fwd subset')
    # (2) adjoint identity ties backward to forward at full size
    lhs = float((y.double() * dy.double()).sum())
    rhs = float((x.double() * dx.double()).sum())
    assert abs(lhs - rhs) <= 1e-6 * float((y.double().abs() * dy.double().abs()).sum())
    # (3) the straightforward kernels give the same answers
    abi.set_impl('naive')
    y_n = abi.forward(x, rois, pooled, scale, S)
    assert_parity(y.cpu().numpy(), y_n.cpu().numpy(), FWD_TOL, cfg + ' fwd vs naive')
    del y_n
    dx_n = abi.backward(dy, rois, x.shape, scale, S)
    assert_parity(dx.cpu().numpy(), dx_n.cpu().numpy(), BWD_TOL, cfg + ' bwd vs naive')
    # (4) oracle backward on 32 channel planes of every image (one from each channel block, at
    # varying positions inside it, and the last channel) via the channel-sliced problem
    C = w['data'].shape[1]
    ch = sorted(set([(8 * k + k % 8) % C for k in range(C // 8)] + [C - 1]))
    want_dx = oracle.backward(np.ascontiguousarray(w['dy'][:, ch]), w['rois'],
                              (x.shape[0], len(ch)) + tuple(x.shape[2:]), scale, S, impl='ordered')
    assert_parity(dx[:, ch].cpu().numpy(), want_dx, BWD_TOL, cfg + ' bwd planes')
    # (5) on a constant map every output is the fraction of valid samples, in [0, 1]
    abi.set_impl('auto')
    ones = torch.ones_like(x)
    frac = abi.forward(ones, rois, pooled, scale, S)
    assert float(frac.min()) >= 0 and float(frac.max()) <= 1 + 1e-6
    # (6) run-to-run difference of the backward pass stays inside the tolerance
    dx2 = abi.backward(dy, rois, x.shape, scale, S, assign=True)
    diff = float((dx - dx2).abs().max())
    print('{}: backward run-to-run max abs diff {:.3e} (max |dx| {:.3e})'.format(
        cfg, diff, float(dx.abs().max())), flush=True)
    assert diff <= BWD_TOL * float(dx.abs().max())
    # (7) channels-last tensors at full size: the same numbers as the NCHW entry points
    y_l = abi.forward_nhwc(x.permute(0, 2, 3, 1).contiguous(), rois, pooled, scale, S)
    assert_parity(y_l.permute(0, 3, 1, 2).cpu().numpy(), y.cpu().numpy(), FWD_TOL, cfg + ' fwd channels-last')
    del y_l
    dx_l = abi.backward_nhwc(dy.permute(0, 2, 3, 1).contiguous(), rois,
                             (x.shape[0], x.shape[2], x.shape[3], x.shape[1]), scale, S, assign=True)
    assert_parity(dx_l.permute(0, 3, 1, 2).cpu().numpy(), dx.cpu().numpy(), BWD_TOL, cfg + ' bwd channels-last')


def test_full_size_with_an_adaptive_grid():
    """The cfg2 tensors with sampling_ratio 0 (ceil(bin size) points per bin and axis: merged
    lists in both passes): oracle on a subset of the ROIs (forward) and on eight channel planes
    (backward), the adjoint identity at full size, and the channels-last entry points."""
    w = workloads.make_workload('cfg2')
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], 0
    x, rois, dy = abi.to_dev(w['data']), abi.to_dev(w['rois']), abi.to_dev(w['dy'])
    abi.set_impl('auto')
    native.set_option('kernel_timing', 1)
    try:
        y = abi.forward(x, rois, pooled, scale, S)
        dx = abi.backward(dy, rois, x.shape, scale, S, assign=True)
        assert _last_bracketed_kernel() == 'backward_blocked_kernel'
    finally:
        native.set_option('kernel_timing', 0)
    pick = np.random.default_rng(3).choice(w['rois'].shape[0], 48, replace=False)
    want = oracle.forward(w['data'], w['rois'][pick], pooled, scale, S)
    assert_parity(y[torch.from_numpy(pick).cuda()].cpu().numpy(), want, FWD_TOL, 'fwd subset')
    lhs = float((y.double() * dy.double()).sum())
    rhs = float((x.double() * dx.double()).sum())
    assert abs(lhs - rhs) <= 1e-6 * float((y.double().abs() * dy.double().abs()).sum())
    ch = [0, 37, 70, 103, 136, 169, 202, 255]
    want_dx = oracle.backward(np.ascontiguousarray(w['dy'][:, ch]), w['rois'],
                              (x.shape[0], len(ch)) + tuple(x.shape[2:]), scale, S, impl='ordered')
    assert_parity(dx[:, ch].cpu().numpy(), want_dx, BWD_TOL, 'bwd planes')
    assert torch.equal(dx, abi.backward(dy, rois, x.shape, scale, S, assign=True)), 'repeats bit for bit'
    dx_l = abi.backward_nhwc(dy.permute(0, 2, 3, 1).contiguous(), rois,
                             (x.shape[0], x.shape[2], x.shape[3], x.shape[1]), scale, S, assign=True)
    assert_parity(dx_l.permute(0, 3, 1, 2).cpu().numpy(), dx.cpu().numpy(), BWD_TOL, 'bwd channels-last')


def test_fp16_full_size_subset():
    w = workloads.make_workload('cfg4')
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    x, rois = abi.to_dev(w['data']), abi.to_dev(w['rois'])
    y = abi.forward(x, rois, pooled, scale, S)
    pick = np.random.default_rng(1).choice(w['rois'].shape[0], 32, replace=False)
    want = oracle.forward(w['data'].astype(np.float32), w['rois'][pick], pooled, scale, S)
    got = y[torch.from_numpy(pick).cuda()].float().cpu().numpy()
    assert_parity(got, want.astype(np.float16).astype(np.float32), FP16_TOL, 'cfg4 subset')
