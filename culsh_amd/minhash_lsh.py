"""
MinHash LSH (Jaccard similarity) over sparse binary rows: same public API as
python/culsh/minhash_lsh.py of the reference, running on libculsh_amd.
"""

from __future__ import annotations

from typing import Optional

import numpy as np

from ._culsh_core import Candidates, MinHashCore, MinHashIndex
from .utils import ensure_device_array, get_array_info, resolve_seed


class MinHashLSH:
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

    def __init__(self, n_hash_tables: int, n_hashes: int, seed: Optional[int] = None):
        if n_hash_tables <= 0:
            raise ValueError("n_hash_tables must be positive")
        if n_hashes <= 0:
            raise ValueError("n_hashes must be positive")
        self._n_hash_tables = n_hash_tables
        self._n_hashes = n_hashes
        self._seed = resolve_seed(seed)

    n_hash_tables = property(lambda self: self._n_hash_tables, doc="Number of hash tables.")
    n_hashes = property(lambda self: self._n_hashes, doc="Number of hash functions per hash table.")
    seed = property(lambda self: self._seed, doc="Random seed.")

    def fit(self, X) -> "MinHashLSHModel":
        """Builds the index over the rows of a CSR matrix X (scipy, cupyx or a device CSR
        structure) with int32 indices."""
        n_samples, n_features, _ = get_array_info(X)
        X = ensure_device_array(X)
        indices, indptr = ensure_int32_indices(X)
        core = MinHashCore(self._n_hash_tables, self._n_hashes, self._seed)
        index = core.fit(indices, indptr, n_samples, n_features)
        return MinHashLSHModel(n_hash_tables=self._n_hash_tables, n_hashes=self._n_hashes,
                               n_features=n_features, core=core, index=index)

    def fit_query(self, X) -> Candidates:
        """Candidates of every row of X among the rows of X, with the bucket of each row taken
        from the index build itself (no lookup).  Each row is its own candidate."""
        n_samples, n_features, _ = get_array_info(X)
        X = ensure_device_array(X)
        indices, indptr = ensure_int32_indices(X)
        core = MinHashCore(self._n_hash_tables, self._n_hashes, self._seed)
        return core.fit_query(indices, indptr, n_samples, n_features)


class MinHashLSHModel:
    """Fitted MinHash index plus the core object whose stream later queries run on."""

    def __init__(self, n_hash_tables: int, n_hashes: int, n_features: int, core: MinHashCore, index: MinHashIndex):
        self._n_hash_tables = n_hash_tables
        self._n_hashes = n_hashes
        self._n_features = n_features
        self._core = core
        self._index = index

    n_hash_tables = property(lambda self: self._n_hash_tables, doc="Number of hash tables.")
    n_hashes = property(lambda self: self._n_hashes, doc="Number of hash functions per hash table.")
    n_features = property(lambda self: self._n_features, doc="Number of features.")
    index = property(lambda self: self._index, doc="The fitted index.")

    def query(self, Q) -> Candidates:
        """Candidate neighbours of each row of the CSR matrix Q (n_queries, n_features)."""
        n_queries, n_features, _ = get_array_info(Q)
        Q = ensure_device_array(Q)
        if n_features != self._n_features:
            raise ValueError(f"Query features ({n_features}) != fitted features ({self._n_features})")
        indices, indptr = ensure_int32_indices(Q)
        return self._core.query(indices, indptr, n_queries, self._index)

    def save(self, path: str) -> None:
        """Compressed .npz with the reference's keys (python/culsh/minhash_lsh.py:240-255)."""
        ix = self._index
        np.savez_compressed(
            path,
            n_hash_tables=self._n_hash_tables, n_hashes=self._n_hashes, n_features=self._n_features,
            n_total_candidates=ix.n_total_candidates, n_total_buckets=ix.n_total_buckets, seed=ix.seed,
            sig_nbytes=ix.sig_nbytes,
            candidate_indices=ix.get_candidate_indices(), bucket_signatures=ix.get_bucket_signatures(),
            bucket_candidate_offsets=ix.get_bucket_candidate_offsets(),
            table_bucket_offsets=ix.get_table_bucket_offsets(), hash_a=ix.get_hash_a(), hash_b=ix.get_hash_b(),
        )

    @classmethod
    def load(cls, path: str) -> "MinHashLSHModel":
        """Reads a model written by `save` (or by the reference's MinHashLSHModel.save)."""
        data = np.load(path)
        T, H, d, seed = (int(data[k]) for k in ("n_hash_tables", "n_hashes", "n_features", "seed"))
        core = MinHashCore(n_hash_tables=T, n_hashes=H, seed=seed)
        index = MinHashIndex.load(
            candidate_indices=data["candidate_indices"], bucket_signatures=data["bucket_signatures"],
            bucket_candidate_offsets=data["bucket_candidate_offsets"],
            table_bucket_offsets=data["table_bucket_offsets"], hash_a=data["hash_a"], hash_b=data["hash_b"],
            n_total_candidates=int(data["n_total_candidates"]), n_total_buckets=int(data["n_total_buckets"]),
            n_hash_tables=T, n_hashes=H, sig_nbytes=int(data["sig_nbytes"]), n_features=d, seed=seed,
        )
        return cls(n_hash_tables=T, n_hashes=H, n_features=d, core=core, index=index)


def _np_dtype(arr) -> np.dtype:
    name = str(arr.dtype)
    return np.dtype(name.replace("torch.", "")) if name.startswith("torch.") else np.dtype(arr.dtype)


def ensure_int32_indices(M):
    """(indices, indptr) of a device CSR structure as int32 device arrays; column ids must
    already be int32 (python/culsh/minhash_lsh.py:300-311), row pointers are converted."""
    if _np_dtype(M.indices) != np.int32:
        raise ValueError(f"MinHashLSH requires int32 indices, got {_np_dtype(M.indices)}")
    indptr = M.indptr
    if _np_dtype(indptr) != np.int32:
        indptr = indptr.int() if hasattr(indptr, "int") else indptr.astype(np.int32)
    return M.indices, indptr
