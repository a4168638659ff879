"""Import name of the framework.

The sources live in the folder ``atoma-infer_amd/`` next to this one; a hyphen
cannot appear in a Python module name, so this package points its search path
at that folder and runs its ``__init__`` there.  ``import atoma_infer_amd``
and ``import atoma_infer_amd.engine`` therefore load ``atoma-infer_amd/...``.
"""
import os as _os

_src = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "atoma-infer_amd")
if not _os.path.isdir(_src):  # pragma: no cover - broken checkout
    raise ImportError(f"atoma_infer_amd: source folder not found: {_src}")
__path__.insert(0, _src)
with open(_os.path.join(_src, "__init__.py"), "r", encoding="utf-8") as _f:
    exec(compile(_f.read(), _os.path.join(_src, "__init__.py"), "exec"), globals())
del _os, _f
