"""Import name of the package whose sources live in ``miniserve-llm-nv_amd/``.

The directory name carries a hyphen, which Python cannot import.  This module
loads that directory as the package ``miniserve_amd`` and replaces itself with
it, so ``import miniserve_amd.config`` resolves to
``miniserve-llm-nv_amd/config``.
"""

import importlib.util as _util
import os as _os
import sys as _sys

_PACKAGE_DIR = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "miniserve-llm-nv_amd")
_spec = _util.spec_from_file_location(
    __name__,
    _os.path.join(_PACKAGE_DIR, "__init__.py"),
    submodule_search_locations=[_PACKAGE_DIR],
)
_module = _util.module_from_spec(_spec)
_sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
