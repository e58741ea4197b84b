"""`mobula.op`: `load` publishes an operator module, `register` is the class decorator
operator modules use; every registered operator appears here as `mobula.op.<Name>`
(reference: mobula/op/__init__.py:1-7, mobula/op/register.py)."""
from ..glue import common as _glue_common
from ..glue import register
from .loader import load

# operators registered from now on are added to this namespace by the glue
_glue_common.OP_MODULE_GLOBALS = globals()

__all__ = ['load', 'register']
