"""
`_culsh_core`: the extension-module surface of the reference (python/csrc/bindings.cu:481-588,
stub python/culsh/_culsh_core.pyi), provided here as thin ctypes classes over the C ABI of
libculsh_amd.so.  Class names, method names, argument order, keyword names, return dtypes
and error types match the reference module so that the `culsh` Python layer and its
tests run unchanged on top of it.

Array arguments are any object exposing ``__cuda_array_interface__`` (torch ROCm tensors,
cupy arrays); as in the reference only the device pointer is read
(python/csrc/common/array_utils.cuh:17-28) - shape, dtype and contiguity are the
caller's responsibility.  Work runs on a stream owned by the ``*Core`` object; that
stream synchronises with the null stream, and every method returns after it is idle.

Extra keyword arguments that the reference does not have (`projection=`, `bias=`,
`hash_a=`, `hash_b=` on the fit methods, `as_torch=` on the getters) default to the
reference behaviour.
"""

from __future__ import annotations

import ctypes as C
from typing import Any, Optional

import numpy as np

from . import _lib as L

__all__ = [
    "Candidates",
    "MinHashCore",
    "MinHashIndex",
    "PSLSHCore",
    "PSLSHIndex",
    "RPLSHCore",
    "RPLSHIndex",
]


def _device_pointer(obj: Any) -> int:
    """Device address of a GPU array (python/csrc/common/array_utils.cuh:17-28)."""
    cai = getattr(obj, "__cuda_array_interface__", None)
    if cai is None:
        raise RuntimeError("Expected a device array with __cuda_array_interface__.")
    return int(cai["data"][0])


def _host_ptr(arr: Optional[np.ndarray]):
    return None if arr is None else arr.ctypes.data_as(C.c_void_p)


class _Ctx:
    """Owns a culsh_ctx (stream + scratch arena); shared by a Core and the objects it makes."""

    _default: Optional["_Ctx"] = None

    def __init__(self, device: int = 0):
        self._lib = L.load()
        h = C.c_void_p()
        L.check(self._lib.culsh_ctx_create(device, C.byref(h)))
        self.handle = h

    def __del__(self):
        h = getattr(self, "handle", None)
        if h:
            try:
                self._lib.culsh_ctx_destroy(h)
            except Exception:
                pass
            self.handle = None

    @classmethod
    def default(cls) -> "_Ctx":
        """Context used by objects that are not tied to a Core (loaded indices)."""
        if cls._default is None:
            cls._default = _Ctx(_current_device())
        return cls._default


def _current_device() -> int:
    try:
        import torch

        if torch.cuda.is_available():
            return int(torch.cuda.current_device())
    except Exception:
        pass
    return 0


# --------------------------------------------------------------------------------------
class Candidates:
    """Query result: ascending, duplicate-free candidate row ids per query, flattened,
    with per-query counts and offsets (core/candidates.cuh:14-40)."""

    def __init__(self, handle: C.c_void_p, ctx: _Ctx):
        self._h = handle
        self._ctx = ctx
        self._lib = ctx._lib

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            try:
                self._lib.culsh_candidates_free(h)
            except Exception:
                pass
            self._h = None

    def _meta(self) -> L.CandidatesMeta:
        m = L.CandidatesMeta()
        L.check(self._lib.culsh_candidates_get_meta(self._h, C.byref(m)))
        return m

    def empty(self) -> bool:
        return bool(self._meta().is_empty)

    @property
    def n_queries(self) -> int:
        return int(self._meta().n_queries)

    @property
    def n_total_candidates(self) -> int:
        return int(self._meta().n_total_candidates)

    def _get(self, which: int, n: int, dtype, as_cupy: bool, as_torch: bool):
        # bindings.cu:268-338: an empty object yields a zero-length array of the dtype
        if self.empty():
            n = 0
        if as_cupy:
            import cupy as cp  # optional dependency, exactly as in the reference

            out = cp.empty(n, dtype=dtype)
            if n:
                L.check(self._lib.culsh_candidates_copy_array(
                    self._ctx.handle, self._h, which, _device_pointer(out), out.nbytes, 1))
            return out
        if as_torch:
            import torch

            tdt = {np.int32: torch.int32, np.uint64: torch.int64}[dtype]  # u64 viewed as i64
            out = torch.empty(n, dtype=tdt, device="cuda")
            if n:
                L.check(self._lib.culsh_candidates_copy_array(
                    self._ctx.handle, self._h, which, out.data_ptr(), out.numel() * out.element_size(), 1))
            return out
        out = np.empty(n, dtype=dtype)
        if n:
            L.check(self._lib.culsh_candidates_copy_array(
                self._ctx.handle, self._h, which, _host_ptr(out), out.nbytes, 0))
        return out

    def get_indices(self, as_cupy: bool = False, as_torch: bool = False):
        """int32 [n_total_candidates]"""
        return self._get(L.ARR_QUERY_INDICES, self.n_total_candidates, np.int32, as_cupy, as_torch)

    def get_counts(self, as_cupy: bool = False, as_torch: bool = False):
        """uint64 [n_queries]"""
        return self._get(L.ARR_QUERY_COUNTS, self.n_queries, np.uint64, as_cupy, as_torch)

    def get_offsets(self, as_cupy: bool = False, as_torch: bool = False):
        """uint64 [n_queries + 1]"""
        return self._get(L.ARR_QUERY_OFFSETS, self.n_queries + 1, np.uint64, as_cupy, as_torch)


# --------------------------------------------------------------------------------------
class _IndexBase:
    """Common part of RPLSHIndex / PSLSHIndex / MinHashIndex (bind_core_index_properties,
    bindings.cu:381-404)."""

    _KIND = L.KIND_CORE

    def __init__(self, handle: C.c_void_p, ctx: _Ctx):
        self._h = handle
        self._ctx = ctx
        self._lib = ctx._lib

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            try:
                self._lib.culsh_index_free(h)
            except Exception:
                pass
            self._h = None

    def _meta(self) -> L.IndexMeta:
        m = L.IndexMeta()
        L.check(self._lib.culsh_index_get_meta(self._h, C.byref(m)))
        return m

    def _array(self, which: int, dtype) -> np.ndarray:
        n, es = C.c_uint64(), C.c_uint32()
        L.check(self._lib.culsh_index_array_info(self._h, which, C.byref(n), C.byref(es)))
        out = np.empty(int(n.value), dtype=dtype)
        assert out.itemsize == es.value
        if out.size:
            L.check(self._lib.culsh_index_copy_array(self._ctx.handle, self._h, which, _host_ptr(out), out.nbytes, 0))
        return out

    def empty(self) -> bool:
        m = self._meta()
        return m.n_total_candidates == 0 and m.n_total_buckets == 0 and m.size_bytes == 0

    def size_bytes(self) -> int:
        return int(self._meta().size_bytes)

    n_total_candidates = property(lambda self: int(self._meta().n_total_candidates))
    n_total_buckets = property(lambda self: int(self._meta().n_total_buckets))
    n_hash_tables = property(lambda self: int(self._meta().n_hash_tables))
    n_hashes = property(lambda self: int(self._meta().n_hashes))
    sig_nbytes = property(lambda self: int(self._meta().sig_nbytes))
    n_features = property(lambda self: int(self._meta().n_features))
    seed = property(lambda self: int(self._meta().seed))

    def get_candidate_indices(self) -> np.ndarray:
        return self._array(L.ARR_CANDIDATE_INDICES, np.int32)

    def get_bucket_signatures(self) -> np.ndarray:
        return self._array(L.ARR_BUCKET_SIGNATURES, np.uint8)

    def get_bucket_candidate_offsets(self) -> np.ndarray:
        return self._array(L.ARR_BUCKET_CANDIDATE_OFFSETS, np.int32)

    def get_table_bucket_offsets(self) -> np.ndarray:
        return self._array(L.ARR_TABLE_BUCKET_OFFSETS, np.int32)

    @classmethod
    def _load(cls, is_double: bool, candidate_indices, bucket_signatures, bucket_candidate_offsets,
              table_bucket_offsets, param0, param1, n_total_candidates, n_total_buckets, n_hash_tables,
              n_hashes, sig_nbytes, n_features, seed):
        ctx = _Ctx.default()
        cand = np.ascontiguousarray(candidate_indices, dtype=np.int32)
        bsig = np.ascontiguousarray(bucket_signatures, dtype=np.uint8)
        bco = np.ascontiguousarray(bucket_candidate_offsets, dtype=np.int32)
        tbo = np.ascontiguousarray(table_bucket_offsets, dtype=np.int32)
        if cand.size != n_total_candidates or bco.size != n_total_buckets + 1 or \
                tbo.size != n_hash_tables + 1 or bsig.size != n_total_buckets * sig_nbytes:
            raise RuntimeError("index arrays do not match the index metadata")
        h = C.c_void_p()
        L.check(ctx._lib.culsh_index_load(
            ctx.handle, cls._KIND, int(is_double), _host_ptr(cand), _host_ptr(bsig), _host_ptr(bco),
            _host_ptr(tbo), _host_ptr(param0), _host_ptr(param1), int(n_total_candidates),
            int(n_total_buckets), int(n_hash_tables), int(n_hashes), int(sig_nbytes), int(n_features),
            int(seed), C.byref(h)))
        return cls(h, ctx)


class _DenseIndex(_IndexBase):
    is_double = property(lambda self: bool(self._meta().is_double))

    def _ftype(self):
        return np.float64 if self.is_double else np.float32

    def get_projection_matrix(self) -> np.ndarray:
        """Flat [T*H*n_features] in the index precision (bindings.cu:369-373)."""
        return self._array(L.ARR_PROJECTION, self._ftype())


class RPLSHIndex(_DenseIndex):
    _KIND = L.KIND_RPLSH

    @staticmethod
    def _load_typed(dtype, candidate_indices, bucket_signatures, bucket_candidate_offsets, table_bucket_offsets,
                    projection, n_total_candidates, n_total_buckets, n_hash_tables, n_hashes, sig_nbytes,
                    n_features, seed) -> "RPLSHIndex":
        proj = np.ascontiguousarray(projection, dtype=dtype).reshape(-1)
        if proj.size != n_hash_tables * n_hashes * n_features:
            raise RuntimeError("projection does not match the index metadata")
        return RPLSHIndex._load(dtype == np.float64, candidate_indices, bucket_signatures,
                                bucket_candidate_offsets, table_bucket_offsets, proj, None, n_total_candidates,
                                n_total_buckets, n_hash_tables, n_hashes, sig_nbytes, n_features, seed)

    @staticmethod
    def load_float(candidate_indices, bucket_signatures, bucket_candidate_offsets, table_bucket_offsets,
                   projection, n_total_candidates, n_total_buckets, n_hash_tables, n_hashes, sig_nbytes,
                   n_features, seed) -> "RPLSHIndex":
        return RPLSHIndex._load_typed(np.float32, candidate_indices, bucket_signatures, bucket_candidate_offsets,
                                      table_bucket_offsets, projection, n_total_candidates, n_total_buckets,
                                      n_hash_tables, n_hashes, sig_nbytes, n_features, seed)

    @staticmethod
    def load_double(candidate_indices, bucket_signatures, bucket_candidate_offsets, table_bucket_offsets,
                    projection, n_total_candidates, n_total_buckets, n_hash_tables, n_hashes, sig_nbytes,
                    n_features, seed) -> "RPLSHIndex":
        return RPLSHIndex._load_typed(np.float64, candidate_indices, bucket_signatures, bucket_candidate_offsets,
                                      table_bucket_offsets, projection, n_total_candidates, n_total_buckets,
                                      n_hash_tables, n_hashes, sig_nbytes, n_features, seed)


class PSLSHIndex(_DenseIndex):
    _KIND = L.KIND_PSLSH

    def get_bias(self) -> np.ndarray:
        return self._array(L.ARR_BIAS, self._ftype())

    @staticmethod
    def _load_typed(dtype, candidate_indices, bucket_signatures, bucket_candidate_offsets, table_bucket_offsets,
                    projection, bias, n_total_candidates, n_total_buckets, n_hash_tables, n_hashes, sig_nbytes,
                    n_features, seed) -> "PSLSHIndex":
        proj = np.ascontiguousarray(projection, dtype=dtype).reshape(-1)
        b = np.ascontiguousarray(bias, dtype=dtype).reshape(-1)
        if proj.size != n_hash_tables * n_hashes * n_features or b.size != n_hash_tables * n_hashes:
            raise RuntimeError("projection / bias do not match the index metadata")
        return PSLSHIndex._load(dtype == np.float64, candidate_indices, bucket_signatures,
                                bucket_candidate_offsets, table_bucket_offsets, proj, b, n_total_candidates,
                                n_total_buckets, n_hash_tables, n_hashes, sig_nbytes, n_features, seed)

    @staticmethod
    def load_float(candidate_indices, bucket_signatures, bucket_candidate_offsets, table_bucket_offsets,
                   projection, bias, n_total_candidates, n_total_buckets, n_hash_tables, n_hashes, sig_nbytes,
                   n_features, seed) -> "PSLSHIndex":
        return PSLSHIndex._load_typed(np.float32, candidate_indices, bucket_signatures, bucket_candidate_offsets,
                                      table_bucket_offsets, projection, bias, n_total_candidates,
                                      n_total_buckets, n_hash_tables, n_hashes, sig_nbytes, n_features, seed)

    @staticmethod
    def load_double(candidate_indices, bucket_signatures, bucket_candidate_offsets, table_bucket_offsets,
                    projection, bias, n_total_candidates, n_total_buckets, n_hash_tables, n_hashes, sig_nbytes,
                    n_features, seed) -> "PSLSHIndex":
        return PSLSHIndex._load_typed(np.float64, candidate_indices, bucket_signatures, bucket_candidate_offsets,
                                      table_bucket_offsets, projection, bias, n_total_candidates,
                                      n_total_buckets, n_hash_tables, n_hashes, sig_nbytes, n_features, seed)


MINHASH_PRIMES = (4294967291, 2147483647)  # the reference's 2^32 - 5 (minhash/hash.cuh:17) and 2^31 - 1


def _check_prime(prime) -> Optional[int]:
    if prime is None:
        return None
    if int(prime) not in MINHASH_PRIMES:
        raise ValueError(f"prime must be one of {MINHASH_PRIMES}, got {prime}")
    return int(prime)


class MinHashIndex(_IndexBase):
    _KIND = L.KIND_MINHASH

    @property
    def prime(self) -> int:
        """The prime the index's hash family is taken modulo (not part of the reference's index, whose
        prime is fixed, minhash/hash.cuh:17)."""
        v = C.c_uint32()
        L.check(self._ctx._lib.culsh_index_minhash_prime(self._h, C.byref(v)))
        return int(v.value)

    def get_hash_a(self) -> np.ndarray:
        return self._array(L.ARR_HASH_A, np.uint32)

    def get_hash_b(self) -> np.ndarray:
        return self._array(L.ARR_HASH_B, np.uint32)

    @staticmethod
    def load(candidate_indices, bucket_signatures, bucket_candidate_offsets, table_bucket_offsets, hash_a, hash_b,
             n_total_candidates, n_total_buckets, n_hash_tables, n_hashes, sig_nbytes, n_features,
             seed, prime=None) -> "MinHashIndex":
        """`prime` (an addition to bindings.cu:457-476): the prime the saved index was hashed with; None is the
        reference's."""
        a = np.ascontiguousarray(hash_a, dtype=np.uint32).reshape(-1)
        b = np.ascontiguousarray(hash_b, dtype=np.uint32).reshape(-1)
        if a.size != n_hash_tables * n_hashes or b.size != a.size:
            raise RuntimeError("hash_a / hash_b do not match the index metadata")
        ctx = _Ctx.default()  # the context the load below runs on: it hands its prime to the index
        L.check(ctx._lib.culsh_ctx_set_minhash_prime(ctx.handle, _check_prime(prime) or MINHASH_PRIMES[0]))
        try:
            return MinHashIndex._load(False, candidate_indices, bucket_signatures, bucket_candidate_offsets,
                                      table_bucket_offsets, a, b, n_total_candidates, n_total_buckets, n_hash_tables,
                                      n_hashes, sig_nbytes, n_features, seed)
        finally:
            L.check(ctx._lib.culsh_ctx_set_minhash_prime(ctx.handle, MINHASH_PRIMES[0]))


# --------------------------------------------------------------------------------------
class _CoreBase:
    def __init__(self, n_hash_tables: int, n_hashes: int, seed: int = 42):
        self._n_hash_tables = int(n_hash_tables)
        self._n_hashes = int(n_hashes)
        self._seed = int(seed)
        if self._seed < 0 or self._seed >= 1 << 64:
            raise TypeError("seed must fit an unsigned 64-bit integer")
        self._ctx = _Ctx(_current_device())
        self._lib = self._ctx._lib

    n_hash_tables = property(lambda self: self._n_hash_tables)
    n_hashes = property(lambda self: self._n_hashes)
    seed = property(lambda self: self._seed)

    def _param(self, arr, dtype, count: int, name: str):
        if arr is None:
            return None
        a = np.ascontiguousarray(arr, dtype=dtype).reshape(-1)
        if a.size != count:
            raise ValueError(f"{name} must hold {count} values, got {a.size}")
        return a


class _DenseCore(_CoreBase):
    _PREFIX = ""
    _INDEX = _DenseIndex

    def _extra(self):  # arguments between n_hashes and seed
        return ()

    def _params(self, dtype, n_features, projection, bias):
        th = self._n_hash_tables * self._n_hashes
        return (self._param(projection, dtype, th * int(n_features), "projection"),)

    def _fit(self, suffix, dtype, X, n_samples, n_features, projection, bias, query: bool):
        fn = getattr(self._lib, f"culsh_{self._PREFIX}_fit_{'query_' if query else ''}{suffix}")
        params = self._params(dtype, n_features, projection, bias)
        h = C.c_void_p()
        L.check(fn(self._ctx.handle, _device_pointer(X), int(n_samples), int(n_features), self._n_hash_tables,
                   self._n_hashes, *self._extra(), self._seed, *[_host_ptr(p) for p in params], C.byref(h)))
        return Candidates(h, self._ctx) if query else self._INDEX(h, self._ctx)

    def _query(self, suffix, Q, n_queries, index, batch_size):
        fn = getattr(self._lib, f"culsh_{self._PREFIX}_query_{suffix}")
        h = C.c_void_p()
        bs = -1 if batch_size is None else int(batch_size)
        L.check(fn(self._ctx.handle, _device_pointer(Q), int(n_queries), index._h, bs, C.byref(h)))
        return Candidates(h, self._ctx)

    def fit_float(self, X, n_samples, n_features, projection=None, bias=None):
        return self._fit("f32", np.float32, X, n_samples, n_features, projection, bias, False)

    def fit_double(self, X, n_samples, n_features, projection=None, bias=None):
        return self._fit("f64", np.float64, X, n_samples, n_features, projection, bias, False)

    def fit_query_float(self, X, n_samples, n_features, projection=None, bias=None):
        return self._fit("f32", np.float32, X, n_samples, n_features, projection, bias, True)

    def fit_query_double(self, X, n_samples, n_features, projection=None, bias=None):
        return self._fit("f64", np.float64, X, n_samples, n_features, projection, bias, True)

    def query_float(self, Q, n_queries, index, batch_size: Optional[int] = None):
        return self._query("f32", Q, n_queries, index, batch_size)

    def query_double(self, Q, n_queries, index, batch_size: Optional[int] = None):
        return self._query("f64", Q, n_queries, index, batch_size)


class RPLSHCore(_DenseCore):
    """bindings.cu:24-116"""
    _PREFIX = "rplsh"
    _INDEX = RPLSHIndex


class PSLSHCore(_DenseCore):
    """bindings.cu:170-265"""
    _PREFIX = "pslsh"
    _INDEX = PSLSHIndex

    def __init__(self, n_hash_tables: int, n_hashes: int, window_size: int, seed: int = 42):
        super().__init__(n_hash_tables, n_hashes, seed)
        self._window_size = int(window_size)

    window_size = property(lambda self: self._window_size)

    def _extra(self):
        return (self._window_size,)

    def _params(self, dtype, n_features, projection, bias):
        th = self._n_hash_tables * self._n_hashes
        if (projection is None) != (bias is None):
            raise ValueError("projection and bias must be given together")
        return (self._param(projection, dtype, th * int(n_features), "projection"),
                self._param(bias, dtype, th, "bias"))


class MinHashCore(_CoreBase):
    """bindings.cu:118-168.  `prime` is an addition: the prime of the hash family, None = the reference's
    4294967291 (minhash/hash.cuh:17)."""

    def __init__(self, n_hash_tables: int, n_hashes: int, seed: int = 42, prime=None):
        super().__init__(n_hash_tables, n_hashes, seed)
        self._prime = _check_prime(prime) or MINHASH_PRIMES[0]
        L.check(self._lib.culsh_ctx_set_minhash_prime(self._ctx.handle, self._prime))

    prime = property(lambda self: self._prime)

    def _fit(self, indices, indptr, n_samples, n_features, hash_a, hash_b, query: bool):
        th = self._n_hash_tables * self._n_hashes
        if (hash_a is None) != (hash_b is None):
            raise ValueError("hash_a and hash_b must be given together")
        a = self._param(hash_a, np.uint32, th, "hash_a")
        b = self._param(hash_b, np.uint32, th, "hash_b")
        fn = self._lib.culsh_minhash_fit_query if query else self._lib.culsh_minhash_fit
        h = C.c_void_p()
        L.check(fn(self._ctx.handle, _device_pointer(indices), _device_pointer(indptr), int(n_samples),
                   int(n_features), self._n_hash_tables, self._n_hashes, self._seed, _host_ptr(a), _host_ptr(b),
                   C.byref(h)))
        return Candidates(h, self._ctx) if query else MinHashIndex(h, self._ctx)

    def fit(self, indices, indptr, n_samples, n_features, hash_a=None, hash_b=None) -> MinHashIndex:
        return self._fit(indices, indptr, n_samples, n_features, hash_a, hash_b, False)

    def fit_query(self, indices, indptr, n_samples, n_features, hash_a=None, hash_b=None) -> Candidates:
        return self._fit(indices, indptr, n_samples, n_features, hash_a, hash_b, True)

    def query(self, indices, indptr, n_queries, index: MinHashIndex) -> Candidates:
        h = C.c_void_p()
        L.check(self._lib.culsh_minhash_query(self._ctx.handle, _device_pointer(indices), _device_pointer(indptr),
                                              int(n_queries), index._h, C.byref(h)))
        return Candidates(h, self._ctx)
