"""
p-stable LSH (Euclidean distance); public API of python/culsh/pstable_lsh.py of the
reference, running on libculsh_amd.
"""

from __future__ import annotations

from typing import Literal, Optional, Union

import numpy as np

from ._culsh_core import Candidates, PSLSHCore, PSLSHIndex
from ._estimator import Family, LSHEstimator, LSHModel
from .utils import get_logger, is_torch_tensor

_FAMILY = Family(core_cls=PSLSHCore, index_cls=PSLSHIndex, dense=True, hyper=("window_size",),
                 param_arrays=(("projection", "get_projection_matrix"), ("bias", "get_bias")))


class PStableLSHModel(LSHModel):
    """Fitted p-stable index.  `query(Q, batch_size=None)` returns the candidate neighbours of each
    row of Q; `batch_size` bounds peak memory without changing the result."""

    _family = _FAMILY

    def __init__(self, n_hash_tables: int, n_hashes: int, window_size: int, n_features: int, core: PSLSHCore,
                 index: PSLSHIndex):
        self._init_common(core, index, n_hash_tables, n_hashes, n_features, window_size=window_size)

    window_size = property(lambda self: self._hyper["window_size"], doc="Window size.")

    def query(self, Q, batch_size: Optional[int] = None) -> Candidates:
        return self._query(Q, batch_size)


class PStableLSH(LSHEstimator):
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

    _family = _FAMILY
    _model_cls = PStableLSHModel

    def __init__(self, n_hash_tables: int, n_hashes: int, window_size: Union[int, Literal["auto"]] = "auto",
                 seed: Optional[int] = None):
        self._init_common(n_hash_tables, n_hashes, seed)
        if window_size != "auto" and window_size <= 0:
            raise ValueError("window_size must be positive")
        self._window_size: Union[int, Literal["auto"]] = window_size
        self._logger = get_logger(self)

    window_size = property(lambda self: self._window_size, doc="Window size or 'auto' if estimated at fit time.")

    def _hyper_values(self, rows) -> dict:
        w = self._window_size
        if w == "auto":
            w = self._estimate_window_size(rows.device)
            self._logger.info(f"Using estimated window size: {w}")
        return {"window_size": w}

    def fit(self, X) -> PStableLSHModel:
        """Builds the index over the rows of X (float32 or float64) and returns the model."""
        return self._fit(X)

    def fit_query(self, X, batch_size: Optional[int] = None) -> Candidates:
        """Candidates of every row of X among the rows of X; see RPLSH.fit_query for the
        meaning of `batch_size`."""
        return self._fit_query(X, batch_size)

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
