"""Import name of the package that lives in ``tiny-inference-engine_amd/``.

The folder's name is not a Python identifier, so ``import tie_amd`` loads this
file, which puts the folder's package into ``sys.modules`` under this name.
``tie_amd.config``, ``tie_amd.engine`` and the other subpackages then resolve
through the package's search path like those of any package.
"""

import importlib.util
import pathlib
import sys

_folder = pathlib.Path(__file__).resolve().parent / "tiny-inference-engine_amd"
_spec = importlib.util.spec_from_file_location(
    __name__, _folder / "__init__.py", submodule_search_locations=[str(_folder)]
)
_package = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _package
_spec.loader.exec_module(_package)
