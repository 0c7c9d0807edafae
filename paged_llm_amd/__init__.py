"""Importable name of the package whose files live in ``paged-llm_amd/``.

A hyphen cannot appear in an ``import`` statement, so this module points its search path at
that folder and runs the folder's ``__init__.py`` in its own namespace: every submodule is
``paged_llm_amd.<name>`` and is read from ``paged-llm_amd/<name>``.
"""
import os as _os

_real = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "paged-llm_amd")
__path__ = [_real]
with open(_os.path.join(_real, "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(_real, "__init__.py"), "exec"))
del _f
