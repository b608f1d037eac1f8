"""Importable alias of the ``co-rope_amd`` package (a hyphen cannot appear in an ``import`` statement)."""
import importlib
import os
import sys

_root = os.path.dirname(os.path.abspath(__file__))
if _root not in sys.path:
    sys.path.insert(0, _root)
_pkg = importlib.import_module("co-rope_amd")
sys.modules[__name__] = _pkg
# ... and of its submodules, so that ``import corope_amd.rope_attn`` names the module the package's own functions live
# in and not a second copy of it with globals of its own
for _name, _mod in list(sys.modules.items()):
    if _name.startswith("co-rope_amd."):
        sys.modules[__name__ + _name[len("co-rope_amd"):]] = _mod
