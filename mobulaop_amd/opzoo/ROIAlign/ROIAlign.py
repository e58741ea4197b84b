"""ROIAlign operator class (average pooling over a regular sampling grid of
bilinear samples; ROI rows are `[batch_idx, x1, y1, x2, y2]`).

Same constructor, inputs, outputs and write-request handling as the reference
operator (opzoo/ROIAlign/ROIAlign.py:7-51).  One addition: when the gradient is
to be overwritten (`req != add`) and the launcher exports the fused
`roi_align_backward_assign` entry point, the zero-fill of `dx` and the scatter
run as one pass that writes every element of `dx` exactly once.
"""
import numpy as np

import mobulaop_amd as mobula
from mobulaop_amd.const import req


def _numel(t):
    return int(np.prod(t.size())) if callable(t.size) else int(t.size)


@mobula.op.register
class ROIAlign:
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
