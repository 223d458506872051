"""Import shim: makes the folder ``easy_gpt.cpp_amd/`` importable as ``easy_gpt.cpp_amd``.

A folder name with a dot in it cannot be found by the normal import machinery, so
this one-file package loads it by path and registers it under its dotted name.
Everything of substance lives in ``easy_gpt.cpp_amd/``.
"""
import importlib.util as _ilu
import os as _os
import sys as _sys

_root = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "easy_gpt.cpp_amd")
_name = __name__ + ".cpp_amd"
if _name not in _sys.modules:
    _spec = _ilu.spec_from_file_location(
        _name, _os.path.join(_root, "__init__.py"), submodule_search_locations=[_root]
    )
    cpp_amd = _ilu.module_from_spec(_spec)
    _sys.modules[_name] = cpp_amd
    _spec.loader.exec_module(cpp_amd)
else:
    cpp_amd = _sys.modules[_name]
