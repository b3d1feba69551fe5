"""
MinHash LSH (Jaccard similarity) over sparse binary rows; public API of
python/culsh/minhash_lsh.py of the reference, running on libculsh_amd.
"""

from __future__ import annotations

from typing import Optional

from ._culsh_core import MINHASH_PRIMES, Candidates, MinHashCore, MinHashIndex, _check_prime
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

    prime = property(lambda self: self._index.prime, doc="The prime of the hash family.")

    def _extra_fields(self) -> dict:
        # the reference's files name no prime (it has one); the key is written for the other prime only
        return {} if self.prime == MINHASH_PRIMES[0] else {"prime": self.prime}

    @classmethod
    def _extra_kwargs(cls, data) -> dict:
        return {"prime": int(data["prime"])} if "prime" in data.files else {}


class MinHashLSH(LSHEstimator):
    """
    Each row is the set of its non-zero column ids (values are ignored).  A hash of a set is
    min over its members of (a*x + b) mod p, p = 4294967291 as in the reference; two sets agree on one hash with
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
    prime : int, optional
        The prime p of the hash family: 4294967291 (None; the reference's fixed choice,
        cuda/culsh/src/minhash/hash.cuh:17) or 2147483647.  Not a parameter of the reference.

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

    def __init__(self, n_hash_tables: int, n_hashes: int, seed: Optional[int] = None, prime: Optional[int] = None):
        self._init_common(n_hash_tables, n_hashes, seed)
        self._prime = _check_prime(prime)

    prime = property(lambda self: self._prime or MINHASH_PRIMES[0], doc="The prime of the hash family.")

    def _core_kwargs(self) -> dict:
        return {} if self._prime is None else {"prime": self._prime}

    def fit(self, X) -> MinHashLSHModel:
        """Builds the index over the rows of a CSR matrix X (scipy, cupyx or a device CSR
        structure) with int32 indices."""
        return self._fit(X)

    def fit_query(self, X) -> Candidates:
        """Candidates of every row of X among the rows of X, with the bucket of each row taken
        from the index build itself (no lookup).  Each row is its own candidate."""
        return self._fit_query(X)
