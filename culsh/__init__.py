"""
`culsh`: the import name of rishic3/cuLSH's Python package (python/culsh/__init__.py:5-17), served by
culsh_amd.  Callers of the reference run unchanged:

    from culsh import RPLSH, PStableLSH, MinHashLSH
    from culsh.rp_lsh import RPLSHModel
    from culsh._culsh_core import RPLSHCore, Candidates
    from culsh.utils import compute_recall

Every submodule name of the reference resolves to the culsh_amd module of the same name (the very same
module object, so classes compare identical whichever name they were imported under).
"""

import importlib as _importlib
import sys as _sys

import culsh_amd as _impl
from culsh_amd import *  # noqa: F401,F403
from culsh_amd import __all__, __version__  # noqa: F401

for _name in ("_culsh_core", "rp_lsh", "pstable_lsh", "minhash_lsh", "utils", "benchmark"):
    _module = _importlib.import_module(f"culsh_amd.{_name}")
    _sys.modules[f"{__name__}.{_name}"] = _module
    globals()[_name] = _module
del _name, _module
