"""Import name for the package folder `paged-attention-engine_amd/`.

The folder carries the project's name, which is not a Python identifier; this
module loads the folder's `__init__.py` under the importable name
`paged_attention_engine_amd` and makes its sub-packages importable from there.
"""

import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "paged-attention-engine_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
