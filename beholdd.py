"""`import beholdd`: the package in the folder `exec-beholdd_amd/`, under an importable name.

The folder's name has a hyphen, so it cannot follow `import` directly.  This module imports
it once and makes `beholdd` and every `beholdd.<submodule>` the very same module objects, so
that registries and other module state exist once.
"""

import importlib
import os
import sys

_root = os.path.dirname(os.path.abspath(__file__))
if _root not in sys.path:
    sys.path.insert(0, _root)

_REAL = "exec-beholdd_amd"
_package = importlib.import_module(_REAL)
for _name, _module in list(sys.modules.items()):
    if _name == _REAL or _name.startswith(_REAL + "."):
        sys.modules[__name__ + _name[len(_REAL):]] = _module
