"""NumPy glue: operator class -> stateful op object with `__call__/forward` and
`backward(out_grad, in_data, out_data, in_grad, req)`
(reference: mobula/glue/numpy_glue.py).

Host arrays have no device: the function binding hands their pointers to the
launcher with device id -1, and the launcher stages them through GPU memory.
"""
import ctypes

import numpy as np

from .common import (MobulaTensor, INPUT_FUNCS, NPDTYPE2CTYPE, assign, get_in_data,
                     get_in_shape, get_varnames)


class NumPyTensor(MobulaTensor):
    F = np

    @property
    def data_ptr(self):
        a = self.tensor
        if a.flags.c_contiguous:
            return a.ctypes.data_as(ctypes.c_void_p)
        dense = np.ascontiguousarray(a)
        return dense.ctypes.data_as(ctypes.c_void_p), dense

    @property
    def ctype(self):
        return NPDTYPE2CTYPE(self.tensor.dtype)

    @property
    def dev_id(self):
        return None

    @property
    def numel(self):
        return self.tensor.size


def _as_list(value):
    return list(value) if isinstance(value, (list, tuple)) else [value]


def _glue_forward(self, *args, **kwargs):
    inputs, _ = get_in_data(op=self.op, *args, **kwargs)
    self.in_data = inputs
    self.req = ['write'] * len(inputs)
    dtype = inputs[0].dtype
    out_shapes = self.infer_shape(get_in_shape(inputs))[1]
    self.out_data = [np.empty(tuple(int(v) for v in s), dtype=dtype) for s in out_shapes]
    ret = self._forward(*inputs)
    if ret is not None:
        for i, value in enumerate(_as_list(ret)):
            self.assign(self.out_data[i], self.req[i], value)
    return self.out_data[0] if len(self.out_data) == 1 else self.out_data


def _glue_backward(self, out_grad=None, in_data=None, out_data=None, in_grad=None, req=None):
    if in_data is not None:
        self.in_data = in_data
    if out_data is not None:
        self.out_data = out_data
    dtype = self.in_data[0].dtype
    if in_grad is None:
        in_grad = [np.empty_like(d, dtype=dtype) for d in self.in_data]
    self.in_grad = in_grad = _as_list(in_grad)
    if out_grad is None:
        out_grad = [np.ones_like(d, dtype=dtype) for d in self.out_data]
    self.out_grad = out_grad = _as_list(out_grad)
    if req is None:
        req = ['write'] * len(self.in_data)
    assert len(req) == len(self.in_data), ValueError('len(req) should be %d' % len(self.in_data))
    self.req = req
    ret = self._backward(*out_grad)
    if ret is not None:
        ret = _as_list(ret)
        for i in range(len(get_varnames(self._forward))):
            self.assign(in_grad[i], self.req[i], ret[i])
    return in_grad[0] if len(in_grad) == 1 else in_grad


class OpGen(object):
    def __init__(self, op, name):
        self.op = op
        self.name = name
        self.cache = {}

    def __call__(self, *args, **kwargs):
        if self.name not in self.cache:
            self.cache[self.name] = self.register()
        klass = self.cache[self.name]
        if kwargs.pop('__input_type__', None) is not None:
            return klass(*args, **kwargs)  # Op[np.ndarray](**ctor) -> op object
        return klass()(*args, **kwargs)    # Op(arrays...) for ops without ctor args

    def register(self):
        op = self.op
        body = dict(__call__=_glue_forward, forward=_glue_forward, backward=_glue_backward,
                    _forward=op.forward, _backward=op.backward, infer_shape=op.infer_shape,
                    assign=assign, F=property(lambda self: np), op=property(lambda _: op))
        if '__init__' in vars(op):
            body['__init__'] = op.__init__
        body.update(INPUT_FUNCS)
        return type('_%s_NP_OP' % self.name, (op, object), body)


F = np
