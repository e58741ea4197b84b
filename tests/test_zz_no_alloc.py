"""The forward entry point that allocates nothing (roi_align_forward_noalloc_83212f20,
no counterpart in the reference) gives what roi_align_forward_ab78de3c gives:
same kernels, so the comparison is bit for bit.  Two calls in a row through the C
ABI, the second on a smaller problem, both sharing the library's fixed buffer."""
import numpy as np
import pytest
import torch

from mobulaop_amd import abi, native

pytestmark = pytest.mark.gpu


def _problem(seed, N, C, H, W, R, scale):
    rng = np.random.default_rng(seed)
    x = rng.random((N, C, H, W), dtype=np.float32)
    size = np.exp(rng.uniform(np.log(8.0), np.log(0.9 * W / scale), size=(R, 2))).astype(np.float32)
    centre = rng.uniform(0, 1, size=(R, 2)).astype(np.float32) * np.array([W / scale, H / scale], np.float32)
    rois = np.empty((R, 5), np.float32)
    rois[:, 0] = rng.integers(0, N, size=R)
    rois[:, 1:3] = centre - size / 2
    rois[:, 3:5] = centre + size / 2
    return abi.to_dev(x), abi.to_dev(rois)


@pytest.mark.parametrize('S', [2, 0])
def test_two_calls_share_the_fixed_buffer(S):
    lib = native.library()
    assert lib.mobula_hip_roialign_noalloc_init(0) == 48 << 20
    for seed, shape in ((11, (2, 64, 96, 128, 300, 0.25)), (12, (1, 36, 40, 52, 77, 0.125))):
        x, rois = _problem(seed, *shape)
        want = abi.forward(x, rois, (7, 7), shape[5], S)
        y = torch.full_like(want, float('nan'))
        before = native.library().mobula_hip_workspace_bytes()
        abi.forward_noalloc(x, rois, (7, 7), shape[5], S, y=y)
        torch.cuda.synchronize()
        assert native.library().mobula_hip_workspace_bytes() == before   # the thread's workspace was not touched
        assert torch.equal(y, want), (seed, (y - want).abs().max().item())


def test_a_map_beyond_the_fixed_buffer_is_refused():
    # 13 M floats of map: 52 MB of channel-blocked copy, the buffer holds 48 MiB
    x = torch.zeros((1, 256, 200, 256), dtype=torch.float32, device='cuda')
    rois = torch.tensor([[0, 0, 0, 64, 64]], dtype=torch.float32, device='cuda')
    with pytest.raises(RuntimeError, match='fixed'):
        abi.forward_noalloc(x, rois, (7, 7), 0.25, 2)
    # and the next call works (an error belongs to the call that caused it)
    x2, rois2 = _problem(13, 1, 32, 40, 52, 10, 0.25)
    assert torch.equal(abi.forward_noalloc(x2, rois2, (7, 7), 0.25, 2), abi.forward(x2, rois2, (7, 7), 0.25, 2))
