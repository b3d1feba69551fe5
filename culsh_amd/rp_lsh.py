"""
Random-projection LSH (cosine similarity): same public API as python/culsh/rp_lsh.py of the
reference, running on libculsh_amd.
"""

from __future__ import annotations

from typing import Optional

import numpy as np

from ._culsh_core import Candidates, RPLSHCore, RPLSHIndex
from .utils import ensure_device_array, get_array_info, resolve_seed


def _dispatch(dtype, on_f32, on_f64, msg):
    if dtype == np.float32:
        return on_f32
    if dtype == np.float64:
        return on_f64
    raise TypeError(msg)


class RPLSH:
    """
    Sign-of-random-projection hashing into `n_hash_tables` tables of `n_hashes` bits each.
    Two vectors at angle theta agree on one bit with probability 1 - theta/pi, so they share
    a bucket in at least one table with probability 1 - (1 - s^r)^b with s that per-bit
    probability, r = n_hashes (AND) and b = n_hash_tables (OR).

    Parameters
    ----------
    n_hash_tables : int
        Number of hash tables; more tables raise recall and the number of candidates.
    n_hashes : int
        Hash bits per table; more bits make buckets smaller and more precise.
    seed : int, optional
        Seed of the projection matrix. None draws a random seed.

    Examples
    --------
    >>> import numpy as np
    >>> from culsh_amd import RPLSH
    >>> X = np.random.randn(10000, 128).astype(np.float32)
    >>> Q = np.random.randn(100, 128).astype(np.float32)
    >>> model = RPLSH(n_hash_tables=16, n_hashes=8).fit(X)
    >>> cand = model.query(Q)
    >>> cand.get_indices(), cand.get_offsets(), cand.get_counts()
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

    def fit(self, X) -> "RPLSHModel":
        """Builds the index over the rows of X (numpy array, torch tensor or any device array
        of shape (n_samples, n_features), float32 or float64) and returns the model."""
        n_samples, n_features, dtype = get_array_info(X)
        X = ensure_device_array(X)
        core = RPLSHCore(self._n_hash_tables, self._n_hashes, self._seed)
        fit = _dispatch(dtype, core.fit_float, core.fit_double,
                        f"Unsupported dtype: {dtype}. Supported dtypes are float32, float64.")
        index = fit(X, n_samples, n_features)
        return RPLSHModel(n_hash_tables=self._n_hash_tables, n_hashes=self._n_hashes, n_features=n_features,
                          core=core, index=index)

    def fit_query(self, X, batch_size: Optional[int] = None) -> Candidates:
        """Candidates of every row of X among the rows of X (each row is its own candidate).
        Without `batch_size` the bucket of each row is taken from the index build itself,
        which skips the lookup; with `batch_size` this is fit(X) followed by a batched
        query(X), bounding peak memory."""
        if batch_size is not None:
            return self.fit(X).query(X, batch_size=batch_size)
        n_samples, n_features, dtype = get_array_info(X)
        X = ensure_device_array(X)
        core = RPLSHCore(self._n_hash_tables, self._n_hashes, self._seed)
        fq = _dispatch(dtype, core.fit_query_float, core.fit_query_double,
                       f"Unsupported dtype: {dtype}. Supported dtypes are float32, float64.")
        return fq(X, n_samples, n_features)


class RPLSHModel:
    """Fitted RPLSH index plus the core object whose stream later queries run on."""

    def __init__(self, n_hash_tables: int, n_hashes: int, n_features: int, core: RPLSHCore, index: RPLSHIndex):
        self._n_hash_tables = n_hash_tables
        self._n_hashes = n_hashes
        self._n_features = n_features
        self._core = core
        self._index = index

    n_hash_tables = property(lambda self: self._n_hash_tables, doc="Number of hash tables.")
    n_hashes = property(lambda self: self._n_hashes, doc="Number of hashes per hash table.")
    n_features = property(lambda self: self._n_features, doc="Number of features.")
    index = property(lambda self: self._index, doc="The fitted index.")

    def query(self, Q, batch_size: Optional[int] = None) -> Candidates:
        """Candidate neighbours of each row of Q (n_queries, n_features).  `batch_size`
        processes the queries in blocks of that many rows; the result is identical."""
        n_queries, n_features, dtype = get_array_info(Q)
        Q = ensure_device_array(Q)
        if n_features != self._n_features:
            raise ValueError(f"Query features ({n_features}) != fitted features ({self._n_features})")
        query = _dispatch(dtype, self._core.query_float, self._core.query_double,
                          f"Unsupported dtype: {dtype}. Use float32 or float64.")
        return query(Q, n_queries, self._index, batch_size)

    def save(self, path: str) -> None:
        """Writes the model as a compressed .npz with the reference's keys
        (python/culsh/rp_lsh.py:259-274)."""
        ix = self._index
        np.savez_compressed(
            path,
            n_hash_tables=self._n_hash_tables, n_hashes=self._n_hashes, n_features=self._n_features,
            n_total_candidates=ix.n_total_candidates, n_total_buckets=ix.n_total_buckets, seed=ix.seed,
            sig_nbytes=ix.sig_nbytes, is_double=ix.is_double,
            candidate_indices=ix.get_candidate_indices(), bucket_signatures=ix.get_bucket_signatures(),
            bucket_candidate_offsets=ix.get_bucket_candidate_offsets(),
            table_bucket_offsets=ix.get_table_bucket_offsets(), projection=ix.get_projection_matrix(),
        )

    @classmethod
    def load(cls, path: str) -> "RPLSHModel":
        """Reads a model written by `save` (or by the reference's RPLSHModel.save)."""
        data = np.load(path)
        T, H, d, seed = (int(data[k]) for k in ("n_hash_tables", "n_hashes", "n_features", "seed"))
        core = RPLSHCore(n_hash_tables=T, n_hashes=H, seed=seed)
        loader = RPLSHIndex.load_double if data["is_double"] else RPLSHIndex.load_float
        index = loader(
            candidate_indices=data["candidate_indices"], bucket_signatures=data["bucket_signatures"],
            bucket_candidate_offsets=data["bucket_candidate_offsets"],
            table_bucket_offsets=data["table_bucket_offsets"], projection=data["projection"],
            n_total_candidates=int(data["n_total_candidates"]), n_total_buckets=int(data["n_total_buckets"]),
            n_hash_tables=T, n_hashes=H, sig_nbytes=int(data["sig_nbytes"]), n_features=d, seed=seed,
        )
        return cls(n_hash_tables=T, n_hashes=H, n_features=d, core=core, index=index)
