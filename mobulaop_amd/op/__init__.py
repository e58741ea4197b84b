"""`mobula.op`: operator registry and loader
(reference: mobula/op/__init__.py:1-7)."""
__all__ = ['register', 'load']

from .. import glue
glue.common.OP_MODULE_GLOBALS = globals()
from .register import register  # noqa: E402
from .loader import load  # noqa: E402
