"""Importable alias of the package in `turboquant-pytorch_amd/` (a hyphen cannot appear in an
`import` statement).  `import turboquant_amd` gives the very same module object."""
import importlib
import os
import sys

_root = os.path.dirname(os.path.abspath(__file__))
if _root not in sys.path:
    sys.path.insert(0, _root)
_pkg = importlib.import_module("turboquant-pytorch_amd")
sys.modules[__name__] = _pkg
