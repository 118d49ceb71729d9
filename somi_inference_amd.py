"""Import name of the package whose sources live in ``somi-inference_amd/``.

A folder name with a hyphen cannot be written in an ``import`` statement, so
this one-file module loads that folder as the package ``somi_inference_amd``
and puts it in ``sys.modules`` under its own name.  After the first import,
``somi_inference_amd.config`` and the other sub-packages resolve as usual.
"""

import importlib.util
import pathlib
import sys

_dir = pathlib.Path(__file__).resolve().parent / "somi-inference_amd"
_spec = importlib.util.spec_from_file_location(
    __name__, _dir / "__init__.py", submodule_search_locations=[str(_dir)]
)
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
