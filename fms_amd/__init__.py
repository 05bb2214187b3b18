"""Import alias: the package lives in ``foundation-model-stack_amd/``, a folder
name that Python cannot import, so ``import fms_amd`` loads that folder as the
package ``fms_amd``."""

import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "foundation-model-stack_amd")
_spec = importlib.util.spec_from_file_location(
    "fms_amd", os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_module = importlib.util.module_from_spec(_spec)
sys.modules["fms_amd"] = _module
_spec.loader.exec_module(_module)
