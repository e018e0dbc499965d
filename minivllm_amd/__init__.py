"""Import name of the engine.

The sources live in the folder ``mini-vllm_amd/`` at the repository root. A hyphen
cannot appear in a Python module name, so this package only points its search path
at that folder and runs the folder's ``__init__.py`` in its own namespace:
``import minivllm_amd.config`` loads ``mini-vllm_amd/config/``.
"""
import os as _os

_SOURCE_DIR = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "mini-vllm_amd")
if not _os.path.isdir(_SOURCE_DIR):
    raise ImportError(f"engine sources not found at {_SOURCE_DIR}")
__path__ = [_SOURCE_DIR]
_init = _os.path.join(_SOURCE_DIR, "__init__.py")
with open(_init, "r", encoding="utf-8") as _f:
    exec(compile(_f.read(), _init, "exec"))
del _f, _init
