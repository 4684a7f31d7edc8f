"""Import name for the package folder `paged-attention-engine_amd/`.

The folder carries the project's name, which is not a Python identifier; this
module loads the folder's `__init__.py` under the importable name
`paged_attention_engine_amd` and makes its sub-packages importable from there.
`python -m paged_attention_engine_amd ...` runs the command line.
"""

import importlib.util
import os
import sys

_NAME = "paged_attention_engine_amd"


def _load():
    folder = os.path.join(os.path.dirname(os.path.abspath(__file__)), "paged-attention-engine_amd")
    spec = importlib.util.spec_from_file_location(
        _NAME, os.path.join(folder, "__init__.py"), submodule_search_locations=[folder])
    module = importlib.util.module_from_spec(spec)
    sys.modules[_NAME] = module
    spec.loader.exec_module(module)
    return module


if __name__ == "__main__":
    _load()
    from paged_attention_engine_amd.engine.cli import main

    sys.exit(main())
else:
    _load()
