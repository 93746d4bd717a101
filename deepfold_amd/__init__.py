"""Import name of the ``deep-fold_amd/`` source tree.

A hyphen is not legal in a Python module name, so the sources live in
``deep-fold_amd/`` and this package only points its search path there:
``import deepfold_amd.nf4`` loads ``deep-fold_amd/nf4/__init__.py``.
"""

import os as _os

_SRC = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "deep-fold_amd")
if not _os.path.isdir(_SRC):
    raise ImportError(f"deepfold_amd: source tree {_SRC} is missing")
__path__ = [_SRC]

__version__ = "0.1.0"
