"""
culsh_amd: locality-sensitive hashing (random projection, p-stable, MinHash) on AMD
MI355X (gfx950).  The public names are those of the `culsh` package of rishic3/cuLSH; the
compute path is libculsh_amd.so (hand-written HIP kernels behind a C ABI).
"""

from importlib import import_module as _import_module

__version__ = "0.1.0"

# family module -> (estimator, fitted model)
_PUBLIC = {
    "rp_lsh": ("RPLSH", "RPLSHModel"),
    "minhash_lsh": ("MinHashLSH", "MinHashLSHModel"),
    "pstable_lsh": ("PStableLSH", "PStableLSHModel"),
}
__all__ = [name for names in _PUBLIC.values() for name in names]
for _module, _names in _PUBLIC.items():
    _loaded = _import_module(f".{_module}", __name__)
    globals().update({_name: getattr(_loaded, _name) for _name in _names})
del _module, _names, _loaded
