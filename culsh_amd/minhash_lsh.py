"""
MinHash LSH (Jaccard similarity) over sparse binary rows; public API of
python/culsh/minhash_lsh.py of the reference, running on libculsh_amd.
"""

from __future__ import annotations

from typing import Optional

from ._culsh_core import Candidates, MinHashCore, MinHashIndex
from ._estimator import Family, LSHEstimator, LSHModel, ensure_int32_indices  # noqa: F401  (re-exported)

_FAMILY = Family(core_cls=MinHashCore, index_cls=MinHashIndex, dense=False,
                 param_arrays=(("hash_a", "get_hash_a"), ("hash_b", "get_hash_b")))


class MinHashLSHModel(LSHModel):
    """Fitted MinHash index.  `query(Q)` returns the candidate neighbours of each row of the CSR
    matrix Q (n_queries, n_features)."""

    _family = _FAMILY

    def __init__(self, n_hash_tables: int, n_hashes: int, n_features: int, core: MinHashCore, index: MinHashIndex):
        self._init_common(core, index, n_hash_tables, n_hashes, n_features)

    def query(self, Q) -> Candidates:
        return self._query(Q)


class MinHashLSH(LSHEstimator):
    """
    Each row is the set of its non-zero column ids (values are ignored).  A hash of a set is
    min over its members of (a*x + b) mod p, p = 4294967291; two sets agree on one hash with
    probability equal to their Jaccard similarity.  `n_hashes` hashes form a table key and
    `n_hash_tables` tables are probed.

    Parameters
    ----------
    n_hash_tables : int
        Number of hash tables (OR amplification).
    n_hashes : int
        Hash functions per table (AND amplification).
    seed : int, optional
        Seed of the hash coefficients. None draws a random seed.

    Examples
    --------
    >>> import scipy.sparse
    >>> from culsh_amd import MinHashLSH
    >>> X = scipy.sparse.random(10000, 1000, density=0.01, format="csr")
    >>> model = MinHashLSH(n_hash_tables=16, n_hashes=8).fit(X)
    >>> cand = model.query(X[:100])
    """

    _family = _FAMILY
    _model_cls = MinHashLSHModel

    def __init__(self, n_hash_tables: int, n_hashes: int, seed: Optional[int] = None):
        self._init_common(n_hash_tables, n_hashes, seed)

    def fit(self, X) -> MinHashLSHModel:
        """Builds the index over the rows of a CSR matrix X (scipy, cupyx or a device CSR
        structure) with int32 indices."""
        return self._fit(X)

    def fit_query(self, X) -> Candidates:
        """Candidates of every row of X among the rows of X, with the bucket of each row taken
        from the index build itself (no lookup).  Each row is its own candidate."""
        return self._fit_query(X)
