"""
Shared machinery of the three estimator families.

The reference writes fit / fit_query / query / save / load three times over
(python/culsh/{rp_lsh,pstable_lsh,minhash_lsh}.py).  Here a family is described by a small
`Family` record (which core and index classes to use, which extra hyper-parameters it has,
which parameter arrays its index carries), input handling is one of two strategies (dense
rows or CSR rows), and the estimator / model behaviour lives once, in the two base classes
below.  The family modules only add their constructors, doc strings and, for p-stable
hashing, the window estimate.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Optional

import numpy as np

from .utils import ensure_device_array, get_array_info, resolve_seed

# keys every saved model has, in the order the model constructor and the index loaders use them
_INDEX_SCALARS = ("n_total_candidates", "n_total_buckets", "sig_nbytes")
_INDEX_ARRAYS = {
    "candidate_indices": "get_candidate_indices",
    "bucket_signatures": "get_bucket_signatures",
    "bucket_candidate_offsets": "get_bucket_candidate_offsets",
    "table_bucket_offsets": "get_table_bucket_offsets",
}


@dataclass(frozen=True)
class Family:
    """What distinguishes one LSH family from another at the Python level."""

    core_cls: Any
    index_cls: Any
    dense: bool                      # dense float rows (True) or CSR rows (False)
    hyper: tuple = ()                # extra hyper-parameters between n_hashes and seed, e.g. ("window_size",)
    param_arrays: tuple = ()         # (npz key, index getter) of the family's parameter arrays


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


def _typed(core, stem: str, dtype, hint: str) -> Callable:
    """core.<stem>_float or core.<stem>_double for float32 / float64 rows."""
    suffix = {np.dtype(np.float32): "float", np.dtype(np.float64): "double"}.get(np.dtype(dtype))
    if suffix is None:
        raise TypeError(f"Unsupported dtype: {dtype}. {hint}")
    return getattr(core, f"{stem}_{suffix}")


class _Rows:
    """An input matrix made ready for the core: shape, dtype and the device-side arguments."""

    def __init__(self, X, dense: bool):
        self.n_rows, self.n_features, self.dtype = get_array_info(X)
        self.device = ensure_device_array(X)
        self.dense = dense
        if not dense:
            self.indices, self.indptr = ensure_int32_indices(self.device)

    def call(self, core, stem: str, hint: str, *tail):
        if self.dense:
            return _typed(core, stem, self.dtype, hint)(self.device, self.n_rows, *tail)
        return getattr(core, stem)(self.indices, self.indptr, self.n_rows, *tail)


_FIT_HINT = "Supported dtypes are float32, float64."
_QUERY_HINT = "Use float32 or float64."


class LSHEstimator:
    """Unfitted estimator: hyper-parameters plus fit / fit_query."""

    _family: Family
    _model_cls: type

    def _init_common(self, n_hash_tables: int, n_hashes: int, seed: Optional[int]) -> None:
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

    def _hyper_values(self, rows: _Rows) -> dict:
        """Values of the family's extra hyper-parameters for this input (none by default)."""
        return {}

    def _core_for(self, rows: _Rows):
        """The core for this input.  An estimator keeps its last core: fitting again with the same
        settings then reuses the core's stream, scratch memory and seeded hash parameters (the
        reference builds a new core per fit, python/culsh/rp_lsh.py:119-121; the result is the same)."""
        hyper = self._hyper_values(rows)
        extra = self._core_kwargs()
        key = (self._n_hash_tables, self._n_hashes, tuple(hyper[k] for k in self._family.hyper), self._seed,
               tuple(sorted(extra.items())))
        kept = getattr(self, "_kept_core", None)
        if kept is None or kept[0] != key:
            kept = (key, self._family.core_cls(self._n_hash_tables, self._n_hashes, *key[2], self._seed, **extra))
            self._kept_core = kept
        return kept[1], hyper

    def _core_kwargs(self) -> dict:
        """Keyword arguments of the family's core beyond the reference's (none by default)."""
        return {}

    def _fit(self, X):
        rows = _Rows(X, self._family.dense)
        core, hyper = self._core_for(rows)
        index = rows.call(core, "fit", _FIT_HINT, rows.n_features)
        return self._model_cls(n_hash_tables=self._n_hash_tables, n_hashes=self._n_hashes, **hyper,
                               n_features=rows.n_features, core=core, index=index)

    def _fit_query(self, X, batch_size: Optional[int] = None):
        if batch_size is not None:  # fit, then a batched query of the same rows: bounded peak memory
            return self._fit(X).query(X, batch_size=batch_size)
        rows = _Rows(X, self._family.dense)
        core, _ = self._core_for(rows)
        return rows.call(core, "fit_query", _FIT_HINT, rows.n_features)


class LSHModel:
    """Fitted index plus the core object whose stream later queries run on."""

    _family: Family

    def _init_common(self, core, index, n_hash_tables: int, n_hashes: int, n_features: int, **hyper) -> None:
        self._core = core
        self._index = index
        self._n_hash_tables = n_hash_tables
        self._n_hashes = n_hashes
        self._n_features = n_features
        self._hyper = dict(hyper)

    n_hash_tables = property(lambda self: self._n_hash_tables, doc="Number of hash tables.")
    n_hashes = property(lambda self: self._n_hashes, doc="Number of hash functions per hash table.")
    n_features = property(lambda self: self._n_features, doc="Number of features.")
    index = property(lambda self: self._index, doc="The fitted index.")

    def _query(self, Q, batch_size: Optional[int] = None):
        rows = _Rows(Q, self._family.dense)
        if rows.n_features != self._n_features:
            raise ValueError(f"Query features ({rows.n_features}) != fitted features ({self._n_features})")
        tail = (self._index, batch_size) if self._family.dense else (self._index,)
        return rows.call(self._core, "query", _QUERY_HINT, *tail)

    def save(self, path: str) -> None:
        """Writes the model as a compressed .npz whose keys, dtypes and array layouts are those of
        the reference's `save` (python/culsh/rp_lsh.py:259-274, pstable_lsh.py:330-347,
        minhash_lsh.py:240-255), so either implementation loads the other's files."""
        ix, fam = self._index, self._family
        fields = {"n_hash_tables": self._n_hash_tables, "n_hashes": self._n_hashes,
                  "n_features": self._n_features, "seed": ix.seed, **self._hyper}
        fields.update((k, getattr(ix, k)) for k in _INDEX_SCALARS)
        if fam.dense:
            fields["is_double"] = ix.is_double
        fields.update((k, getattr(ix, getter)()) for k, getter in _INDEX_ARRAYS.items())
        fields.update((k, getattr(ix, getter)()) for k, getter in fam.param_arrays)
        fields.update(self._extra_fields())
        np.savez_compressed(path, **fields)

    def _extra_fields(self) -> dict:
        """Keys beyond the reference's that this model has to write to be read back as it is (none by
        default, so that default files hold exactly the reference's keys)."""
        return {}

    @classmethod
    def _extra_kwargs(cls, data) -> dict:
        """Keyword arguments for the core and the index loader from such keys."""
        return {}

    @classmethod
    def load(cls, path: str):
        """Reads a model written by `save` of this package or of the reference."""
        fam = cls._family
        data = np.load(path)
        ints = {k: int(data[k]) for k in ("n_hash_tables", "n_hashes", "n_features", "seed", *fam.hyper)}
        hyper = {k: ints[k] for k in fam.hyper}
        extra = cls._extra_kwargs(data)
        core = fam.core_cls(ints["n_hash_tables"], ints["n_hashes"], *hyper.values(), ints["seed"], **extra)
        if fam.dense:
            loader = fam.index_cls.load_double if data["is_double"] else fam.index_cls.load_float
        else:
            loader = fam.index_cls.load
        arrays = {k: data[k] for k in (*_INDEX_ARRAYS, *(k for k, _ in fam.param_arrays))}
        index = loader(**arrays, **{k: int(data[k]) for k in _INDEX_SCALARS},
                       n_hash_tables=ints["n_hash_tables"], n_hashes=ints["n_hashes"],
                       n_features=ints["n_features"], seed=ints["seed"], **extra)
        return cls(n_hash_tables=ints["n_hash_tables"], n_hashes=ints["n_hashes"], **hyper,
                   n_features=ints["n_features"], core=core, index=index)
