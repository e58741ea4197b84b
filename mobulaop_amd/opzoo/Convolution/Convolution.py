"""Conv2D operator class: y = conv(x, weight) + bias, NCHW input, DCKK weights.

Same constructor, inputs, outputs and shape rules as the reference operator
(opzoo/Convolution/Convolution.py:5-84).  The reference unfolds one image at a
time with im2col and multiplies with the framework's matrix product; here the
forward pass and the three gradients are one launcher call each
(`mobula.func.conv2d_forward / conv2d_backward_data / conv2d_backward_weight /
conv2d_backward_bias`), which run the products on the matrix cores without a
column buffer.  `mobula.func.im2col / col2im` remain available with the
reference's argument lists.
"""
import numpy as np

import mobulaop_amd as mobula
from mobulaop_amd.const import req


def _numel(t):
    return int(np.prod(t.size())) if callable(t.size) else int(t.size)


@mobula.op.register
class Conv2D:
    def __init__(self, channels, kernel_size, strides=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1):
        assert groups == 1, 'grouped convolution is not provided'
        self.channels, self.groups = channels, groups
        self.kernel_size, self.strides = tuple(kernel_size), tuple(strides)
        self.padding, self.dilation = tuple(padding), tuple(dilation)

    def _geometry(self, x_shape):
        N, C, H, W = x_shape
        return (int(N), int(C), int(H), int(W), int(self.channels), self.kernel_size[0], self.kernel_size[1],
                self.padding[0], self.padding[1], self.strides[0], self.strides[1],
                self.dilation[0], self.dilation[1])

    def forward(self, x, weight, bias=None):
        if self.req[0] == req.null:
            return
        out = self.y if self.req[0] != req.add else self.F.empty_like(self.y)
        mobula.func.conv2d_forward(_numel(out), x, weight, bias if bias is not None else weight,
                                   0 if bias is None else 1, *self._geometry(x.shape), out)
        if self.req[0] == req.add:
            self.y[:] += out

    def backward(self, dy):
        x, weight = self.X[0], self.X[1]
        geometry = self._geometry(x.shape)
        if self.req[0] != req.null:
            mobula.func.conv2d_backward_data(_numel(self.dX[0]), dy, weight, int(self.req[0] == req.add),
                                             *geometry, self.dX[0])
        if self.req[1] != req.null:
            mobula.func.conv2d_backward_weight(_numel(self.dX[1]), dy, x, int(self.req[1] == req.add),
                                               *geometry, self.dX[1])
        if len(self.X) == 3 and self.req[2] != req.null:
            mobula.func.conv2d_backward_bias(_numel(self.dX[2]), dy, int(self.req[2] == req.add),
                                             int(dy.shape[0]), int(dy.shape[2] * dy.shape[3]), self.dX[2])

    def infer_shape(self, in_shape):
        """[x (N,C,H,W), weight (D,C,KH,KW), optional bias (D,)] -> y (N,D,OH,OW) with
        O = (size + 2*pad - dilated kernel) // stride + 1 on each axis."""
        assert len(in_shape) in (2, 3), \
            "The inputs should be feature map(NCHW layout), weight and bias(optional)"
        x, weight = in_shape[0], in_shape[1]
        assert len(x) == 4, "input: NCHW"
        assert len(weight) == 4, "weight: DCKK"
        assert len(in_shape) == 2 or len(in_shape[2]) == 1, "bias: D"
        expected = (self.channels, x[1]) + tuple(self.kernel_size)
        assert tuple(weight) == expected, "weight: expected {}, got {}".format(expected, tuple(weight))
        out = []
        for axis in (0, 1):
            reach = self.dilation[axis] * (self.kernel_size[axis] - 1) + 1   # extent of the dilated kernel
            out.append((x[2 + axis] + 2 * self.padding[axis] - reach) // self.strides[axis] + 1)
        return in_shape, [(x[0], self.channels, out[0], out[1])]
