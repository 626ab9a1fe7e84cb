"""Import alias: ``import crosslayer_coding_amd`` gives the package that lives in the
directory ``crosslayer-coding_amd/`` (a hyphen is not a valid identifier)."""

import importlib
import sys

_REAL = "crosslayer-coding_amd"
_pkg = importlib.import_module(_REAL)
for _name, _mod in list(sys.modules.items()):
    if _name.startswith(_REAL + "."):
        sys.modules[__name__ + _name[len(_REAL):]] = _mod
sys.modules[__name__] = _pkg
