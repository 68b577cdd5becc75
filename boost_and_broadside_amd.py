"""Import alias for the package directory ``boost-and-broadside_amd``.

The directory name is not a Python identifier, so ``import boost_and_broadside_amd``
resolves to this file, which loads the directory's ``__init__.py`` under this module
name and lets submodule imports (``boost_and_broadside_amd.ops`` ...) find their files.
"""

import importlib.util as _util
import os as _os
import sys as _sys

_dir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "boost-and-broadside_amd")
_spec = _util.spec_from_file_location(
    __name__, _os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_module = _util.module_from_spec(_spec)
_sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
