"""Import shim: the package lives in the directory ``nengo-ocl_amd/``.

A hyphen is not legal in a Python module name, so this one-file module makes
``import nengo_ocl_amd`` resolve to that directory: it sets ``__path__`` so
that the import machinery treats this module as a package rooted there, then
runs the package's ``__init__.py`` in this namespace.
"""

import os as _os

_pkg_dir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "nengo-ocl_amd")
__path__ = [_pkg_dir]
__file__ = _os.path.join(_pkg_dir, "__init__.py")
__package__ = __name__  # relative imports inside the package's __init__ resolve against it
if __spec__ is not None:
    __spec__.submodule_search_locations = __path__

with open(__file__, "r", encoding="utf-8") as _f:
    exec(compile(_f.read(), __file__, "exec"))  # noqa: S102
del _f, _os
