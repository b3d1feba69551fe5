"""
Random-projection LSH (cosine similarity); public API of python/culsh/rp_lsh.py of the
reference, running on libculsh_amd.
"""

from __future__ import annotations

from typing import Optional

from ._culsh_core import Candidates, RPLSHCore, RPLSHIndex
from ._estimator import Family, LSHEstimator, LSHModel

_FAMILY = Family(core_cls=RPLSHCore, index_cls=RPLSHIndex, dense=True,
                 param_arrays=(("projection", "get_projection_matrix"),))


class RPLSHModel(LSHModel):
    """Fitted RPLSH index.  `query(Q, batch_size=None)` returns the candidate neighbours of each
    row of Q (n_queries, n_features); with `batch_size` the queries are processed in blocks of
    that many rows and the result is identical."""

    _family = _FAMILY

    def __init__(self, n_hash_tables: int, n_hashes: int, n_features: int, core: RPLSHCore, index: RPLSHIndex):
        self._init_common(core, index, n_hash_tables, n_hashes, n_features)

    def query(self, Q, batch_size: Optional[int] = None) -> Candidates:
        return self._query(Q, batch_size)


class RPLSH(LSHEstimator):
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

    _family = _FAMILY
    _model_cls = RPLSHModel

    def __init__(self, n_hash_tables: int, n_hashes: int, seed: Optional[int] = None):
        self._init_common(n_hash_tables, n_hashes, seed)

    def fit(self, X) -> RPLSHModel:
        """Builds the index over the rows of X (numpy array, torch tensor or any device array
        of shape (n_samples, n_features), float32 or float64) and returns the model."""
        return self._fit(X)

    def fit_query(self, X, batch_size: Optional[int] = None) -> Candidates:
        """Candidates of every row of X among the rows of X (each row is its own candidate).
        Without `batch_size` the bucket of each row is taken from the index build itself,
        which skips the lookup; with `batch_size` this is fit(X) followed by a batched
        query(X), bounding peak memory."""
        return self._fit_query(X, batch_size)
