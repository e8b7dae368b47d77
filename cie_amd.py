"""Import name of the package that lives in ``cloud-inference-from-scratch_amd/``.

The folder carries the upstream project's name, which is no Python identifier;
this module loads the folder as the package ``cie_amd`` so that
``import cie_amd.engine`` and relative imports inside the folder work.
"""

import importlib.util
import os
import sys

_folder = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cloud-inference-from-scratch_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_folder, "__init__.py"), submodule_search_locations=[_folder]
)
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
