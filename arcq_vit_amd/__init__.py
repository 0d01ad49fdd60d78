"""Import shim: the package sources live in the directory ``arcq-vit_amd/`` (whose
name is not a valid Python identifier).  This module makes them importable as
``arcq_vit_amd`` by pointing the package search path there and running that
directory's ``__init__.py`` in this module's namespace."""
import os as _os

_real = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "arcq-vit_amd")
__path__ = [_real]
with open(_os.path.join(_real, "__init__.py"), "r", encoding="utf-8") as _f:
    exec(compile(_f.read(), _os.path.join(_real, "__init__.py"), "exec"))
del _f
