"""Import alias: the package directory is `self-forcing_amd/` (not a Python identifier);
`import self_forcing_amd` gives the same package object, and
`from self_forcing_amd.monarch_attn import ...` the same sub-module objects."""
import importlib
import os
import sys

_root = os.path.dirname(os.path.abspath(__file__))
if _root not in sys.path:
    sys.path.insert(0, _root)
_real = "self-forcing_amd"
_pkg = importlib.import_module(_real)
for _name, _mod in list(sys.modules.items()):
    if _name.startswith(_real + "."):
        sys.modules[__name__ + _name[len(_real):]] = _mod
sys.modules[__name__] = _pkg
