"""
ctypes loader for libculsh_oracle.so (the C restatement in culsh_oracle.c).

TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg may import this module.  It returns the same dataclasses as culsh_oracle.py so
the two restatements can be compared field by field.
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

from . import culsh_oracle as npo

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libculsh_oracle.so")


class _Index(C.Structure):
    _fields_ = [
        ("all_candidate_indices", C.POINTER(C.c_int32)),
        ("all_bucket_signatures", C.POINTER(C.c_uint8)),
        ("bucket_candidate_offsets", C.POINTER(C.c_int32)),
        ("table_bucket_offsets", C.POINTER(C.c_int32)),
        ("item_to_bucket", C.POINTER(C.c_int32)),
        ("n_total_candidates", C.c_int32),
        ("n_total_buckets", C.c_int32),
        ("n_hash_tables", C.c_int32),
        ("n_hashes", C.c_int32),
        ("sig_nbytes", C.c_int32),
    ]


class _Candidates(C.Structure):
    _fields_ = [
        ("query_candidate_indices", C.POINTER(C.c_int32)),
        ("query_candidate_counts", C.POINTER(C.c_uint64)),
        ("query_candidate_offsets", C.POINTER(C.c_uint64)),
        ("n_queries", C.c_int32),
        ("n_total_candidates", C.c_uint64),
        ("n_raw_candidates", C.c_uint64),
    ]


def build(force: bool = False) -> str:
    """Compile the C oracle in place (gcc + OpenMP)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(f"{_LIB_PATH} is not built; run `make -C oracle`")
        _lib = C.CDLL(_LIB_PATH)
        _lib.oracle_num_threads.restype = C.c_int
    return _lib


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _copy(ptr, n, dtype):
    if n == 0:
        return np.zeros(0, dtype=dtype)
    return np.ctypeslib.as_array(ptr, shape=(n,)).astype(dtype, copy=True)


def rplsh_hash(X: np.ndarray, P: np.ndarray, T: int, H: int, blocked: bool = False) -> np.ndarray:
    """`blocked` (fp32): the cache- and vector-blocked form, bit-identical to the plain one."""
    n, d = X.shape
    sig = np.empty((T, n, H), dtype=np.uint8)
    X = np.ascontiguousarray(X)
    P = np.ascontiguousarray(P, dtype=X.dtype)
    fn = lib().oracle_rplsh_hash_f32 if X.dtype == np.float32 else lib().oracle_rplsh_hash_f64
    if blocked and X.dtype == np.float32:
        fn = lib().oracle_rplsh_hash_f32_blocked
    fn(_p(X), _p(P), n, d, T, H, _p(sig))
    return sig


def pslsh_hash(X: np.ndarray, P: np.ndarray, b: np.ndarray, T: int, H: int) -> np.ndarray:
    n, d = X.shape
    sig = np.empty((T, n, H), dtype=np.int32)
    X = np.ascontiguousarray(X)
    P = np.ascontiguousarray(P, dtype=X.dtype)
    b = np.ascontiguousarray(b, dtype=X.dtype)
    fn = lib().oracle_pslsh_hash_f32 if X.dtype == np.float32 else lib().oracle_pslsh_hash_f64
    fn(_p(X), _p(P), _p(b), n, d, T, H, _p(sig))
    return sig


def minhash_hash(indices, indptr, A, B, T: int, H: int, prime: int = 4294967291) -> np.ndarray:
    n = len(indptr) - 1
    sig = np.empty((T, n, H), dtype=np.uint32)
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    indptr = np.ascontiguousarray(indptr, dtype=np.int32)
    A = np.ascontiguousarray(A, dtype=np.uint32)
    B = np.ascontiguousarray(B, dtype=np.uint32)
    lib().oracle_minhash_mod(_p(indices), _p(indptr), _p(A), _p(B), n, T, H, C.c_uint64(prime), _p(sig))
    return sig


class CIndex:
    """Owns an oracle_index; `.to_numpy()` copies it into the numpy oracle's dataclass."""

    def __init__(self):
        self.s = _Index()

    def __del__(self):
        try:
            lib().oracle_index_free(C.byref(self.s))
        except Exception:
            pass

    def to_numpy(self, n: int) -> npo.Index:
        s = self.s
        N, B, T, S = s.n_total_candidates, s.n_total_buckets, s.n_hash_tables, s.sig_nbytes
        itb = _copy(s.item_to_bucket, n * T, np.int32) if s.item_to_bucket else None
        return npo.Index(
            _copy(s.all_candidate_indices, N, np.int32),
            _copy(s.all_bucket_signatures, B * S, np.uint8),
            _copy(s.bucket_candidate_offsets, B + 1, np.int32),
            _copy(s.table_bucket_offsets, T + 1, np.int32),
            N, B, T, s.n_hashes, S, itb)


def _sig_bytes(X_sig: np.ndarray):
    T, n = X_sig.shape[0], X_sig.shape[1]
    b = np.ascontiguousarray(X_sig).view(np.uint8).reshape(T, n, -1)
    return b, T, n, b.shape[2]


def fit_index_c(X_sig: np.ndarray, n_hashes: int, with_item_to_bucket: bool = False) -> CIndex:
    b, T, n, S = _sig_bytes(X_sig)
    ix = CIndex()
    rc = lib().oracle_fit_index(_p(b), n, T, n_hashes, S, int(with_item_to_bucket), C.byref(ix.s))
    if rc:
        raise MemoryError("oracle_fit_index")
    return ix


def fit_index(X_sig: np.ndarray, n_hashes: int, with_item_to_bucket: bool = False) -> npo.Index:
    return fit_index_c(X_sig, n_hashes, with_item_to_bucket).to_numpy(X_sig.shape[1])


def _cands_to_numpy(c: _Candidates) -> npo.Candidates:
    out = npo.Candidates(
        _copy(c.query_candidate_indices, c.n_total_candidates, np.int32),
        _copy(c.query_candidate_counts, c.n_queries, np.uint64),
        _copy(c.query_candidate_offsets, c.n_queries + 1, np.uint64),
        c.n_queries, int(c.n_total_candidates))
    out.n_raw_candidates = int(c.n_raw_candidates)
    lib().oracle_candidates_free(C.byref(c))
    return out


def query_index_c(Q_sig: np.ndarray, ix: CIndex, keep: bool = True):
    """Runs the C query; returns the numpy dataclass (keep=True) or only (U, R) totals."""
    b, T, nq, S = _sig_bytes(Q_sig)
    c = _Candidates()
    rc = lib().oracle_query_index(_p(b), nq, S, C.byref(ix.s), C.byref(c))
    if rc:
        raise MemoryError("oracle_query_index")
    if keep:
        return _cands_to_numpy(c)
    tot = (int(c.n_total_candidates), int(c.n_raw_candidates))
    lib().oracle_candidates_free(C.byref(c))
    return tot


def fit_query(X_sig: np.ndarray, n_hashes: int) -> npo.Candidates:
    b, T, n, S = _sig_bytes(X_sig)
    c = _Candidates()
    rc = lib().oracle_fit_query(_p(b), n, T, n_hashes, S, C.byref(c))
    if rc:
        raise MemoryError("oracle_fit_query")
    return _cands_to_numpy(c)
