"""Import name of the package that lives in the folder ``infinicore-infer_amd/``.

The folder name is not a Python identifier, so this module stands in for it:
it points ``__path__`` at the folder and runs the folder's ``__init__.py`` in
its own namespace.  ``import infinicore_infer_amd.config`` then resolves to
``infinicore-infer_amd/config/``.
"""
import os as _os

__path__ = [_os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "infinicore-infer_amd")]
_init = _os.path.join(__path__[0], "__init__.py")
with open(_init, "r", encoding="utf-8") as _f:
    exec(compile(_f.read(), _init, "exec"))
del _f, _init
