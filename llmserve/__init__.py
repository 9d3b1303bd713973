"""Import name of the engine in a checkout.

The sources live in the folder ``llmserve-triton-kernels_amd`` beside this one; that
folder's name is not a Python identifier, so this package maps its own submodule
search path onto it and runs that folder's ``__init__.py`` as its own: ``import llmserve.engine``
loads ``llmserve-triton-kernels_amd/engine``, and ``python -m llmserve.cli`` is the command line.
(An installed copy needs none of this: pyproject.toml installs that folder as ``llmserve``.)
"""

import os as _os

_SOURCE_DIR = _os.path.join(
    _os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "llmserve-triton-kernels_amd"
)
__path__ = [_SOURCE_DIR]
with open(_os.path.join(_SOURCE_DIR, "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(_SOURCE_DIR, "__init__.py"), "exec"), globals())
