"""Framework glue: turns an operator class into a torch autograd module or a
NumPy op object (reference: mobula/glue/__init__.py:1-4)."""
from . import common
from . import backend
from .common import register, register_cstruct, CUSTOM_OP_LIST

common.backend = backend
