"""PyTorch (ROCm) glue: operator class -> autograd.Function + nn.Module
(reference: mobula/glue/torch_glue.py).

Differences from the reference, on purpose:
  * gradients are always written into fresh tensors (the reference reuses an
    existing `.grad` as scratch, which double-counts when autograd then
    accumulates the returned tensor into that same `.grad`);
  * `torch.float16` is a known element type (fp16-storage forward);
  * `current_stream()` lets the function binding launch on torch's stream
    instead of synchronising the device around every call.
"""
import ctypes

import torch

from .common import (MobulaTensor, INPUT_FUNCS, assign, get_in_data, get_in_shape,
                     get_varnames)
from ..dtype import c_bfloat16, c_half

# int32 / float32 / float64 are the reference's (mobula/glue/torch_glue.py:6-9); the
# other widths follow the NumPy glue
THDTYPE2CTYPE_MAP = {
    torch.int32: ctypes.c_int,
    torch.float32: ctypes.c_float,
    torch.float64: ctypes.c_double,
    torch.float16: c_half,
    torch.bfloat16: c_bfloat16,
    torch.int8: ctypes.c_int8,
    torch.int16: ctypes.c_int16,
    torch.int64: ctypes.c_int64,
}


class TorchTensor(MobulaTensor):
    F = torch

    @property
    def data_ptr(self):
        t = self.tensor
        if t.is_contiguous():
            return ctypes.c_void_p(t.data_ptr())
        dense = t.contiguous()
        return ctypes.c_void_p(dense.data_ptr()), dense

    @property
    def ctype(self):
        ctype = THDTYPE2CTYPE_MAP.get(self.tensor.dtype)
        assert ctype is not None, TypeError('Unknown Type: {}'.format(self.tensor.dtype))
        return ctype

    @property
    def dev_id(self):
        dev = self.tensor.device
        return None if dev.type == 'cpu' else dev.index

    @property
    def numel(self):
        return self.tensor.numel()


def current_stream(dev_id):
    """Raw hipStream_t of torch's current stream on `dev_id` (as an int)."""
    return torch.cuda.current_stream(dev_id).cuda_stream


def _make_function(op, op_name):
    def forward(ctx, mod, *inputs):
        ctx.mod = mod
        mod.in_data = inputs
        mod.req = ['write'] * len(inputs)
        out_shapes = mod.infer_shape(get_in_shape(inputs))[1]
        dtype = inputs[0].dtype if inputs else torch.float32
        device = inputs[0].device if inputs else torch.device('cpu')
        # an operator that says so gets 4-D outputs in the memory format of a channels-last first input
        fmt = torch.contiguous_format
        if (getattr(mod, 'follows_channels_last', False) and inputs and inputs[0].dim() == 4 and
                not inputs[0].is_contiguous() and inputs[0].is_contiguous(memory_format=torch.channels_last)):
            fmt = torch.channels_last
        mod.out_data = [torch.empty(tuple(int(v) for v in s), dtype=dtype, device=device,
                                    memory_format=fmt if len(s) == 4 else torch.contiguous_format)
                        for s in out_shapes]
        ret = mod._forward(*inputs)
        if ret is not None:
            ret = ret if isinstance(ret, (list, tuple)) else [ret]
            for i, value in enumerate(ret):
                mod.assign(mod.out_data[i], mod.req[i], value)
        return mod.out_data[0] if len(mod.out_data) == 1 else tuple(mod.out_data)

    def backward(ctx, *out_grads):
        mod = ctx.mod
        dtype = mod.in_data[0].dtype if mod.in_data else torch.float32
        mod.in_grad = [torch.empty_like(d, dtype=dtype) for d in mod.in_data]
        mod.out_grad = out_grads
        mod.req = ['write'] * len(mod.in_data)
        ret = mod._backward(*out_grads)
        if ret is not None:
            ret = ret if isinstance(ret, (list, tuple)) else [ret]
            for i in range(len(get_varnames(mod._forward))):
                mod.assign(mod.in_grad[i], mod.req[i], ret[i])
        # the operator object lets go of the gradients: a tensor that autograd alone
        # holds is adopted as .grad, one that is still referenced here is copied first
        grads = tuple(mod.in_grad)
        mod.in_grad = mod.out_grad = None
        return (None,) + grads

    return type('_%s_TORCH_FUNC' % op_name, (op, torch.autograd.Function),
                dict(forward=staticmethod(forward), backward=staticmethod(backward)))


def _make_module(op, op_name, func):
    def __init__(self, *args, **kwargs):
        torch.nn.Module.__init__(self)
        op.__init__(self, *args, **kwargs)

    def forward(self, *inputs):
        return func.apply(self, *inputs)

    body = dict(__init__=__init__, forward=forward, _forward=op.forward,
                _backward=op.backward, assign=assign, F=property(lambda self: torch))
    body.update(INPUT_FUNCS)
    return type('_%s_TORCH_NN_MODULE' % op_name, (op, torch.nn.Module), body)


class OpGen(object):
    def __init__(self, op, name):
        self.op = op
        self.name = name
        self.cache = {}

    def __call__(self, *args, **kwargs):
        if self.name not in self.cache:
            self.cache[self.name] = self.register()
        inputs, (ctor_args, ctor_kwargs) = get_in_data(op=self.op, *args, **kwargs)
        return self.cache[self.name](*ctor_args, **ctor_kwargs)(*inputs)

    def register(self):
        return _make_module(self.op, self.name, _make_function(self.op, self.name))
