"""The raw C-ABI helpers live in the package (mobulaop_amd/abi.py); tests use them under this name."""
from mobulaop_amd.abi import *   # noqa: F401,F403
from mobulaop_amd.abi import _begin, _end, _geom, _ptr   # noqa: F401
