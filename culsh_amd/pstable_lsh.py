"""
p-stable LSH (Euclidean distance): same public API as python/culsh/pstable_lsh.py of the
reference, running on libculsh_amd.
"""

from __future__ import annotations

from typing import Literal, Optional, Union

import numpy as np

from ._culsh_core import Candidates, PSLSHCore, PSLSHIndex
from .rp_lsh import _dispatch
from .utils import ensure_device_array, get_array_info, get_logger, is_torch_tensor, resolve_seed


class PStableLSH:
    """
    Hashes h(x) = floor((a.x + b) / w) with a ~ N(0, I) and b ~ U(0, w]; `n_hashes` of them
    form one table key and `n_hash_tables` tables are probed.  Nearby points (in L2) fall
    into the same window with a probability that grows with `window_size`.

    Parameters
    ----------
    n_hash_tables : int
        Number of hash tables (OR amplification).
    n_hashes : int
        Hashes per table (AND amplification).
    window_size : int or "auto"
        Quantisation width w.  "auto" takes the mean L2 norm of (a sample of) the rows at
        fit time, truncated to an integer and at least 1.
    seed : int, optional
        Seed of the projections and offsets. None draws a random seed.

    Examples
    --------
    >>> import numpy as np
    >>> from culsh_amd import PStableLSH
    >>> X = np.random.randn(10000, 128).astype(np.float32)
    >>> model = PStableLSH(n_hash_tables=16, n_hashes=8, window_size=4).fit(X)
    >>> cand = model.query(X[:100])
    """

    def __init__(self, n_hash_tables: int, n_hashes: int, window_size: Union[int, Literal["auto"]] = "auto",
                 seed: Optional[int] = None):
        if n_hash_tables <= 0:
            raise ValueError("n_hash_tables must be positive")
        if n_hashes <= 0:
            raise ValueError("n_hashes must be positive")
        if window_size != "auto" and window_size <= 0:
            raise ValueError("window_size must be positive")
        self._n_hash_tables = n_hash_tables
        self._n_hashes = n_hashes
        self._window_size: Union[int, Literal["auto"]] = window_size
        self._seed = resolve_seed(seed)
        self._logger = get_logger(self)

    n_hash_tables = property(lambda self: self._n_hash_tables, doc="Number of hash tables.")
    n_hashes = property(lambda self: self._n_hashes, doc="Number of hash functions per hash table.")
    window_size = property(lambda self: self._window_size, doc="Window size or 'auto' if estimated at fit time.")
    seed = property(lambda self: self._seed, doc="Random seed.")

    def _resolve_window(self, X) -> int:
        if self._window_size != "auto":
            return self._window_size
        w = self._estimate_window_size(X)
        self._logger.info(f"Using estimated window size: {w}")
        return w

    def fit(self, X) -> "PStableLSHModel":
        """Builds the index over the rows of X (float32 or float64) and returns the model."""
        n_samples, n_features, dtype = get_array_info(X)
        X = ensure_device_array(X)
        window_size = self._resolve_window(X)
        core = PSLSHCore(self._n_hash_tables, self._n_hashes, window_size, self._seed)
        fit = _dispatch(dtype, core.fit_float, core.fit_double,
                        f"Unsupported dtype: {dtype}. Supported dtypes are float32, float64.")
        index = fit(X, n_samples, n_features)
        return PStableLSHModel(n_hash_tables=self._n_hash_tables, n_hashes=self._n_hashes,
                               window_size=window_size, n_features=n_features, core=core, index=index)

    def fit_query(self, X, batch_size: Optional[int] = None) -> Candidates:
        """Candidates of every row of X among the rows of X; see RPLSH.fit_query for the
        meaning of `batch_size`."""
        if batch_size is not None:
            return self.fit(X).query(X, batch_size=batch_size)
        n_samples, n_features, dtype = get_array_info(X)
        X = ensure_device_array(X)
        window_size = self._resolve_window(X)
        core = PSLSHCore(self._n_hash_tables, self._n_hashes, window_size, self._seed)
        fq = _dispatch(dtype, core.fit_query_float, core.fit_query_double,
                       f"Unsupported dtype: {dtype}. Supported dtypes are float32, float64.")
        return fq(X, n_samples, n_features)

    @staticmethod
    def _estimate_window_size(X, scale_factor: float = 1.0, max_samples: int = 10000) -> int:
        """max(1, int(mean row L2 norm / scale_factor)) over at most `max_samples` rows drawn
        without replacement (python/culsh/pstable_lsh.py:191-223)."""
        n_samples = len(X)
        if is_torch_tensor(X):
            import torch

            Xs = X[torch.randperm(n_samples, device=X.device)[:max_samples]] if n_samples > max_samples else X
            mean_magnitude = float(torch.linalg.norm(Xs.double(), dim=1).mean())
        elif hasattr(X, "__cuda_array_interface__"):
            import cupy as cp

            Xs = X[cp.random.choice(n_samples, max_samples, replace=False)] if n_samples > max_samples else X
            mean_magnitude = float(cp.linalg.norm(Xs, axis=1).mean())
        else:
            X = np.asarray(X)
            Xs = X[np.random.choice(n_samples, max_samples, replace=False)] if n_samples > max_samples else X
            mean_magnitude = float(np.linalg.norm(Xs, axis=1).mean())
        return max(1, int(mean_magnitude / scale_factor))


class PStableLSHModel:
    """Fitted p-stable index plus the core object whose stream later queries run on."""

    def __init__(self, n_hash_tables: int, n_hashes: int, window_size: int, n_features: int, core: PSLSHCore,
                 index: PSLSHIndex):
        self._n_hash_tables = n_hash_tables
        self._n_hashes = n_hashes
        self._window_size = window_size
        self._n_features = n_features
        self._core = core
        self._index = index

    n_hash_tables = property(lambda self: self._n_hash_tables, doc="Number of hash tables.")
    n_hashes = property(lambda self: self._n_hashes, doc="Number of hashes per hash table.")
    window_size = property(lambda self: self._window_size, doc="Window size.")
    n_features = property(lambda self: self._n_features, doc="Number of features.")
    index = property(lambda self: self._index, doc="The fitted index.")

    def query(self, Q, batch_size: Optional[int] = None) -> Candidates:
        """Candidate neighbours of each row of Q; `batch_size` bounds peak memory."""
        n_queries, n_features, dtype = get_array_info(Q)
        Q = ensure_device_array(Q)
        if n_features != self._n_features:
            raise ValueError(f"Query features ({n_features}) != fitted features ({self._n_features})")
        query = _dispatch(dtype, self._core.query_float, self._core.query_double,
                          f"Unsupported dtype: {dtype}. Use float32 or float64.")
        return query(Q, n_queries, self._index, batch_size)

    def save(self, path: str) -> None:
        """Compressed .npz with the reference's keys (python/culsh/pstable_lsh.py:330-347)."""
        ix = self._index
        np.savez_compressed(
            path,
            n_hash_tables=self._n_hash_tables, n_hashes=self._n_hashes, window_size=self._window_size,
            n_features=self._n_features, n_total_candidates=ix.n_total_candidates,
            n_total_buckets=ix.n_total_buckets, seed=ix.seed, sig_nbytes=ix.sig_nbytes, is_double=ix.is_double,
            candidate_indices=ix.get_candidate_indices(), bucket_signatures=ix.get_bucket_signatures(),
            bucket_candidate_offsets=ix.get_bucket_candidate_offsets(),
            table_bucket_offsets=ix.get_table_bucket_offsets(), projection=ix.get_projection_matrix(),
            bias=ix.get_bias(),
        )

    @classmethod
    def load(cls, path: str) -> "PStableLSHModel":
        """Reads a model written by `save` (or by the reference's PStableLSHModel.save)."""
        data = np.load(path)
        T, H, d, seed, w = (int(data[k]) for k in ("n_hash_tables", "n_hashes", "n_features", "seed", "window_size"))
        core = PSLSHCore(n_hash_tables=T, n_hashes=H, window_size=w, seed=seed)
        loader = PSLSHIndex.load_double if data["is_double"] else PSLSHIndex.load_float
        index = loader(
            candidate_indices=data["candidate_indices"], bucket_signatures=data["bucket_signatures"],
            bucket_candidate_offsets=data["bucket_candidate_offsets"],
            table_bucket_offsets=data["table_bucket_offsets"], projection=data["projection"], bias=data["bias"],
            n_total_candidates=int(data["n_total_candidates"]), n_total_buckets=int(data["n_total_buckets"]),
            n_hash_tables=T, n_hashes=H, sig_nbytes=int(data["sig_nbytes"]), n_features=d, seed=seed,
        )
        return cls(n_hash_tables=T, n_hashes=H, window_size=w, n_features=d, core=core, index=index)
