"""
culsh_amd: locality-sensitive hashing (random projection, p-stable, MinHash) on AMD
MI355X (gfx950).  Same public API as the `culsh` package of rishic3/cuLSH; the compute
path is libculsh_amd.so (hand-written HIP kernels behind a C ABI).
"""

from .minhash_lsh import MinHashLSH, MinHashLSHModel
from .pstable_lsh import PStableLSH, PStableLSHModel
from .rp_lsh import RPLSH, RPLSHModel

__version__ = "0.1.0"
__all__ = [
    "RPLSH",
    "RPLSHModel",
    "MinHashLSH",
    "MinHashLSHModel",
    "PStableLSH",
    "PStableLSHModel",
]
