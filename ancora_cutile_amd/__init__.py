"""Importable alias of the package directory `ancora-cutile_amd/` (a hyphen cannot appear
in a Python module name): the package search path points at that directory and its
__init__ runs here, so `import ancora_cutile_amd.adamw` loads `ancora-cutile_amd/adamw.py`."""
import os as _os

_real = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))),
                      "ancora-cutile_amd")
__path__ = [_real]
with open(_os.path.join(_real, "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(_real, "__init__.py"), "exec"))
