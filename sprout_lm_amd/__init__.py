"""Import name of the engine whose sources live in the folder `sprout-lm_amd/`.

A hyphen cannot stand in a Python module name, so this package only extends
its search path to that folder and then runs the real `__init__` from there.
"""
import os as _os

_SRC = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "sprout-lm_amd")
__path__.insert(0, _SRC)
with open(_os.path.join(_SRC, "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(_SRC, "__init__.py"), "exec"))
del _f
