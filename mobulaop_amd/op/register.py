"""`@mobula.op.register` (reference: mobula/op/register.py)."""
from .. import glue


def register(*args, **kwargs):
    return glue.register(*args, **kwargs)
