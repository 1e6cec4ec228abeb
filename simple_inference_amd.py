"""Import name for the package that lives in the folder ``simple-inference_amd/``.

The folder name carries a hyphen and so cannot be written in an ``import``
statement.  Importing ``simple_inference_amd`` runs this file, which loads the
folder's ``__init__.py`` as a package under this module's name and puts it in
``sys.modules`` in its own place; ``import simple_inference_amd.config`` and the
like then resolve through the package's ``__path__`` as usual.
"""

import importlib.util
import os
import sys

_here = os.path.dirname(os.path.abspath(__file__))
_pkg_dir = os.path.join(_here, "simple-inference_amd")

_spec = importlib.util.spec_from_file_location(
    __name__,
    os.path.join(_pkg_dir, "__init__.py"),
    submodule_search_locations=[_pkg_dir],
)
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
