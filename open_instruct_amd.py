"""Import shim: the package directory is named ``open-instruct_amd`` (not a valid Python
identifier), so ``import open_instruct_amd`` lands here and this module replaces itself with the
package loaded from that directory."""

import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "open-instruct_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_mod = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _mod
_spec.loader.exec_module(_mod)
