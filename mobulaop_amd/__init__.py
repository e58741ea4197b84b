"""MI355X-native ROIAlign behind MobulaOP's Python surface.

`import mobulaop_amd as mobula` gives the part of the `mobula` API the ROIAlign
path uses: `mobula.op.load`, `mobula.op.register`, `mobula.op.<Op>`,
`mobula.func.<kernel>`, `mobula.glue`, `mobula.config`, `mobula.testing`.
Unless another package of that name is already imported, this package is also
published as `mobula` in `sys.modules`, so operator files and scripts written
for MobulaOP (`import mobula`) run unchanged.
"""
import sys as _sys

from .version import __version__
from .config import config
from . import glue
from . import func
from . import op
from . import testing

function = func
operator = op

_sys.modules.setdefault('mobula', _sys.modules[__name__])
for _sub in ('func', 'op', 'glue', 'config', 'testing', 'const'):
    if 'mobula.' + _sub not in _sys.modules and _sys.modules['mobula'] is _sys.modules[__name__]:
        from importlib import import_module as _imp
        _sys.modules['mobula.' + _sub] = _imp('.' + _sub, __name__)
