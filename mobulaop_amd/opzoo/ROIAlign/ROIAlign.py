"""ROIAlign operator class (average pooling over a regular sampling grid of
bilinear samples; ROI rows are `[batch_idx, x1, y1, x2, y2]`).

Same constructor, inputs, outputs and write-request handling as the reference
operator (opzoo/ROIAlign/ROIAlign.py:7-51).  One addition: when the gradient is
to be overwritten (`req != add`) and the launcher exports the fused
`roi_align_backward_assign` entry point, the zero-fill of `dx` and the scatter
run as one pass that writes every element of `dx` exactly once.  A second one:
torch tensors in `torch.channels_last` format on a GPU are handed to the
channels-last entry points as they are (no conversion to NCHW, and none inside
the library), when the launcher takes the shape.
"""
import numpy as np

import mobulaop_amd as mobula
from mobulaop_amd import native
from mobulaop_amd.const import req


def _numel(t):
    return int(np.prod(t.size())) if callable(t.size) else int(t.size)


def _is_channels_last(t):
    """A 4-D torch GPU tensor laid out as [N,H,W,C] (and not also as [N,C,H,W])."""
    try:
        import torch
    except ImportError:
        return False
    return (isinstance(t, torch.Tensor) and t.dim() == 4 and t.device.type != 'cpu' and
            not t.is_contiguous() and t.is_contiguous(memory_format=torch.channels_last))


def _nhwc(t):
    """The [N,H,W,C] view of a channels-last [N,C,H,W] tensor (contiguous)."""
    return t.permute(0, 2, 3, 1)


@mobula.op.register
class ROIAlign:
    follows_channels_last = True   # the torch glue allocates y in the memory format of data

    def __init__(self, pooled_size, spatial_scale, sampling_ratio):
        self.pooled_size = pooled_size
        self.spatial_scale = spatial_scale
        self.sampling_ratio = sampling_ratio

    def forward(self, data, rois):
        if self.req[0] == req.null:
            return
        geometry = (self.spatial_scale, data.shape[1], data.shape[2], data.shape[3],
                    self.pooled_size[0], self.pooled_size[1], self.sampling_ratio)
        out = self.y
        if (self.req[0] != req.add and _is_channels_last(data) and _is_channels_last(out) and
                hasattr(mobula.func, 'roi_align_forward_nhwc') and
                native.roialign_channels_last_supported(False, data.element_size(), data.shape[1], data.shape[2],
                                                        data.shape[3], self.pooled_size, self.sampling_ratio,
                                                        rois.shape[0])):
            mobula.func.roi_align_forward_nhwc(_numel(out), _nhwc(data), *geometry, rois, _nhwc(out))
            return
        if self.req[0] == req.add:
            fresh = self.F.empty_like(out)
            mobula.func.roi_align_forward(_numel(out), data, *geometry, rois, fresh)
            self.y[:] += fresh
        else:
            mobula.func.roi_align_forward(_numel(out), data, *geometry, rois, out)

    def backward(self, dy):
        if self.req[0] == req.null:
            return
        data, rois = self.X
        geometry = (self.spatial_scale, data.shape[1], data.shape[2], data.shape[3],
                    self.pooled_size[0], self.pooled_size[1], self.sampling_ratio)
        dx = self.dX[0]
        if (self.req[0] != req.add and _is_channels_last(data) and _is_channels_last(dx) and
                hasattr(mobula.func, 'roi_align_backward_nhwc_assign') and
                native.roialign_channels_last_supported(True, dx.element_size(), data.shape[1], data.shape[2],
                                                        data.shape[3], self.pooled_size, self.sampling_ratio,
                                                        rois.shape[0])):
            import torch
            dy_cl = dy.contiguous(memory_format=torch.channels_last)
            try:
                mobula.func.roi_align_backward_nhwc_assign(_numel(dy), _nhwc(dy_cl), *geometry, int(data.shape[0]),
                                                           _nhwc(dx), rois)
                taken = True
            except RuntimeError:
                # Sampling grids other than 1 or 2 points are merged into lists whose size
                # depends on the boxes: an adaptive grid of more than 2^15 points per bin, or
                # a stream that is being captured (the size comes back through a blocking
                # copy), is refused there.  The NCHW entry point below takes every grid.
                if self.sampling_ratio in (1, 2):
                    raise
                taken = False
            if taken:
                if self.req[1] not in (req.null, req.add):
                    self.dX[1][:] = 0
                return
        fused = getattr(mobula.func, 'roi_align_backward_assign', None)
        if self.req[0] != req.add and fused is not None:
            fused(_numel(dy), dy, *geometry, int(data.shape[0]), self.dX[0], rois)
        else:
            if self.req[0] != req.add:
                self.dX[0][:] = 0
            mobula.func.roi_align_backward(_numel(dy), dy, *geometry, self.dX[0], rois)
        if self.req[1] not in (req.null, req.add):
            self.dX[1][:] = 0  # no gradient flows to the boxes

    def infer_shape(self, in_shape):
        dshape, rshape = in_shape
        assert len(dshape) == 4
        assert len(rshape) == 2
        assert rshape[1] == 5
        oshape = [rshape[0], dshape[1], self.pooled_size[0], self.pooled_size[1]]
        return [dshape, rshape], [oshape]
