"""
Thin ctypes driver of libculsh_amd.so's C ABI: a context object whose methods call the entry
points with numpy arrays (copied to device memory through torch tensors) and hand results back
as numpy arrays.  Nothing here computes results - it only moves arrays in and out.  Used by the
benchmark, the smoke run and the tests; the estimator classes go through `_culsh_core` instead.
"""

from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L


def torch():
    import torch as t

    return t


def dev(arr: np.ndarray):
    """numpy -> device tensor (uint32/uint64 go through a same-width signed view)."""
    t = torch()
    a = np.ascontiguousarray(arr)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    elif a.dtype == np.uint64:
        a = a.view(np.int64)
    if a.size == 0:
        return t.empty(0, dtype=t.from_numpy(np.zeros(1, a.dtype)).dtype, device="cuda")
    return t.from_numpy(a).cuda()


def ptr(tensor) -> int:
    return 0 if tensor is None else int(tensor.data_ptr())


def hp(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class Ctx:
    def __init__(self, device: int = 0):
        self.lib = L.load()
        self.h = C.c_void_p()
        L.check(self.lib.culsh_ctx_create(device, C.byref(self.h)))

    def close(self):
        if self.h:
            self.lib.culsh_ctx_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def set_minhash_prime(self, prime: int) -> None:
        """The prime MinHash fits, loads and `minhash_compute` calls of this context hash with from now on."""
        L.check(self.lib.culsh_ctx_set_minhash_prime(self.h, prime))

    def index_minhash_prime(self, ih) -> int:
        v = C.c_uint32()
        L.check(self.lib.culsh_index_minhash_prime(ih, C.byref(v)))
        return int(v.value)

    # ------------------------------------------------------------ objects
    def index_arrays(self, ih):
        """dict with the four core arrays + metadata of an index handle."""
        m = L.IndexMeta()
        L.check(self.lib.culsh_index_get_meta(ih, C.byref(m)))
        out = {f: getattr(m, f) for f, _ in L.IndexMeta._fields_}
        for name, which, dt in (("all_candidate_indices", L.ARR_CANDIDATE_INDICES, np.int32),
                                ("all_bucket_signatures", L.ARR_BUCKET_SIGNATURES, np.uint8),
                                ("bucket_candidate_offsets", L.ARR_BUCKET_CANDIDATE_OFFSETS, np.int32),
                                ("table_bucket_offsets", L.ARR_TABLE_BUCKET_OFFSETS, np.int32)):
            n, es = C.c_uint64(), C.c_uint32()
            L.check(self.lib.culsh_index_array_info(ih, which, C.byref(n), C.byref(es)))
            a = np.empty(n.value, dtype=dt)
            L.check(self.lib.culsh_index_copy_array(self.h, ih, which, hp(a), a.nbytes, 0))
            out[name] = a
        return out

    def index_param(self, ih, which, dtype):
        n, es = C.c_uint64(), C.c_uint32()
        L.check(self.lib.culsh_index_array_info(ih, which, C.byref(n), C.byref(es)))
        a = np.empty(n.value, dtype=dtype)
        assert a.itemsize == es.value
        if a.size:
            L.check(self.lib.culsh_index_copy_array(self.h, ih, which, hp(a), a.nbytes, 0))
        return a

    def candidates_arrays(self, ch, free: bool = True):
        m = L.CandidatesMeta()
        L.check(self.lib.culsh_candidates_get_meta(ch, C.byref(m)))
        idx = np.empty(m.n_total_candidates, dtype=np.int32)
        cnt = np.empty(m.n_queries, dtype=np.uint64)
        off = np.empty(m.n_queries + 1, dtype=np.uint64)
        for a, which in ((idx, L.ARR_QUERY_INDICES), (cnt, L.ARR_QUERY_COUNTS), (off, L.ARR_QUERY_OFFSETS)):
            L.check(self.lib.culsh_candidates_copy_array(self.h, ch, which, hp(a), a.nbytes, 0))
        if free:
            self.lib.culsh_candidates_free(ch)
        return {"indices": idx, "counts": cnt, "offsets": off, "n_queries": m.n_queries,
                "n_total_candidates": int(m.n_total_candidates), "is_empty": bool(m.is_empty)}

    def candidates_meta(self, ch):
        m = L.CandidatesMeta()
        L.check(self.lib.culsh_candidates_get_meta(ch, C.byref(m)))
        return {"n_queries": m.n_queries, "n_total_candidates": int(m.n_total_candidates), "is_empty": bool(m.is_empty)}

    def candidates_merge(self, acc, other):
        """Candidates::merge: appends `other` (consumed) to `acc` (a handle or None); returns the new handle."""
        h = C.c_void_p(acc.value if acc is not None else None)
        L.check(self.lib.culsh_candidates_merge(self.h, C.byref(h), other))
        return h

    def candidates_device_ptr(self, ch, which) -> int:
        return int(self.lib.culsh_candidates_device_ptr(ch, which) or 0)

    def stream(self) -> int:
        return int(self.lib.culsh_ctx_stream(self.h) or 0)

    def synchronize(self) -> None:
        L.check(self.lib.culsh_ctx_synchronize(self.h))

    # ------------------------------------------------------------ stage level
    def rplsh_hash(self, X: np.ndarray, P: np.ndarray, T: int, H: int) -> np.ndarray:
        n, d = X.shape
        t = torch()
        sig = t.empty(T * n * H, dtype=t.uint8, device="cuda")
        fn = self.lib.culsh_rplsh_hash_f32 if X.dtype == np.float32 else self.lib.culsh_rplsh_hash_f64
        dX, dP = dev(X), dev(np.ascontiguousarray(P, dtype=X.dtype))
        L.check(fn(self.h, ptr(dX), ptr(dP), n, d, T, H, ptr(sig)))
        return sig.cpu().numpy().reshape(T, n, H)

    def pslsh_hash(self, X, P, b, T, H) -> np.ndarray:
        n, d = X.shape
        t = torch()
        sig = t.empty(T * n * H, dtype=t.int32, device="cuda")
        fn = self.lib.culsh_pslsh_hash_f32 if X.dtype == np.float32 else self.lib.culsh_pslsh_hash_f64
        dX, dP, db = dev(X), dev(np.ascontiguousarray(P, dtype=X.dtype)), dev(np.ascontiguousarray(b, dtype=X.dtype))
        L.check(fn(self.h, ptr(dX), ptr(dP), ptr(db), n, d, T, H, ptr(sig)))
        return sig.cpu().numpy().reshape(T, n, H)

    def minhash_compute(self, indices, indptr, A, B, T, H) -> np.ndarray:
        n = len(indptr) - 1
        t = torch()
        sig = t.empty(T * n * H, dtype=t.int32, device="cuda")
        di, dp = dev(indices.astype(np.int32)), dev(indptr.astype(np.int32))
        dA, dB = dev(A.astype(np.uint32)), dev(B.astype(np.uint32))
        L.check(self.lib.culsh_minhash_compute(self.h, ptr(di), ptr(dp), ptr(dA), ptr(dB), n, T, H, ptr(sig)))
        return sig.cpu().numpy().view(np.uint32).reshape(T, n, H)

    @staticmethod
    def _sig_bytes(sig: np.ndarray):
        T, n = sig.shape[0], sig.shape[1]
        b = np.ascontiguousarray(sig).view(np.uint8).reshape(T, n, -1)
        return b, T, n, b.shape[2]

    def core_fit_index(self, sig: np.ndarray, H: int, want_item_to_bucket: bool = False):
        b, T, n, S = self._sig_bytes(sig)
        t = torch()
        dsig = dev(b.reshape(-1))
        itb = t.empty(n * T, dtype=t.int32, device="cuda") if want_item_to_bucket else None
        ih = C.c_void_p()
        L.check(self.lib.culsh_core_fit_index(self.h, ptr(dsig), n, T, H, S, ptr(itb) or None, C.byref(ih)))
        return ih, (itb.cpu().numpy() if itb is not None else None)

    def core_query_index(self, qsig: np.ndarray, ih, as_handle: bool = False):
        b, T, nq, S = self._sig_bytes(qsig)
        dsig = dev(b.reshape(-1))
        ch = C.c_void_p()
        L.check(self.lib.culsh_core_query_index(self.h, ptr(dsig), nq, S, ih, C.byref(ch)))
        return ch if as_handle else self.candidates_arrays(ch)

    def core_find_matching_buckets(self, qsig: np.ndarray, ih, static: bool = False) -> np.ndarray:
        """`static`: through the entry point that allocates nothing (asynchronous: synchronised here)."""
        b, T, nq, S = self._sig_bytes(qsig)
        t = torch()
        dsig = dev(b.reshape(-1))
        m = t.empty(nq * T, dtype=t.int32, device="cuda")
        if static:
            L.check(self.lib.culsh_core_find_matching_buckets_static(self.h, ptr(dsig), nq, S, ih, ptr(m)))
            self.synchronize()
        else:
            L.check(self.lib.culsh_core_find_matching_buckets(self.h, ptr(dsig), nq, S, ih, ptr(m)))
        return m.cpu().numpy()

    def core_query_from_matched(self, matched: np.ndarray, nq: int, ih):
        dm = dev(matched.astype(np.int32))
        ch = C.c_void_p()
        L.check(self.lib.culsh_core_query_from_matched_buckets(self.h, ptr(dm), nq, ih, C.byref(ch)))
        return self.candidates_arrays(ch)

    def core_fit_query(self, sig: np.ndarray, H: int):
        b, T, n, S = self._sig_bytes(sig)
        dsig = dev(b.reshape(-1))
        ch = C.c_void_p()
        L.check(self.lib.culsh_core_fit_query(self.h, ptr(dsig), n, T, H, S, C.byref(ch)))
        return self.candidates_arrays(ch)

    def free_index(self, ih):
        self.lib.culsh_index_free(ih)

    # ------------------------------------------------------------ family level
    def rplsh_fit(self, X, T, H, seed=42, P=None):
        n, d = X.shape
        sfx = "f32" if X.dtype == np.float32 else "f64"
        dX = dev(X)
        Pc = None if P is None else np.ascontiguousarray(P, dtype=X.dtype)
        ih = C.c_void_p()
        L.check(getattr(self.lib, f"culsh_rplsh_fit_{sfx}")(self.h, ptr(dX), n, d, T, H, seed, hp(Pc), C.byref(ih)))
        return ih

    def rplsh_query(self, Q, ih, batch_size=-1):
        nq = Q.shape[0]
        sfx = "f32" if Q.dtype == np.float32 else "f64"
        dQ = dev(Q)
        ch = C.c_void_p()
        L.check(getattr(self.lib, f"culsh_rplsh_query_{sfx}")(self.h, ptr(dQ), nq, ih, batch_size, C.byref(ch)))
        return self.candidates_arrays(ch)

    def rplsh_fit_query(self, X, T, H, seed=42, P=None):
        n, d = X.shape
        sfx = "f32" if X.dtype == np.float32 else "f64"
        dX = dev(X)
        Pc = None if P is None else np.ascontiguousarray(P, dtype=X.dtype)
        ch = C.c_void_p()
        L.check(getattr(self.lib, f"culsh_rplsh_fit_query_{sfx}")(self.h, ptr(dX), n, d, T, H, seed, hp(Pc), C.byref(ch)))
        return self.candidates_arrays(ch)

    def pslsh_fit(self, X, T, H, w, seed=42, P=None, b=None):
        n, d = X.shape
        sfx = "f32" if X.dtype == np.float32 else "f64"
        dX = dev(X)
        Pc = None if P is None else np.ascontiguousarray(P, dtype=X.dtype)
        bc = None if b is None else np.ascontiguousarray(b, dtype=X.dtype)
        ih = C.c_void_p()
        L.check(getattr(self.lib, f"culsh_pslsh_fit_{sfx}")(self.h, ptr(dX), n, d, T, H, w, seed, hp(Pc), hp(bc), C.byref(ih)))
        return ih

    def pslsh_query(self, Q, ih, batch_size=-1):
        nq = Q.shape[0]
        sfx = "f32" if Q.dtype == np.float32 else "f64"
        dQ = dev(Q)
        ch = C.c_void_p()
        L.check(getattr(self.lib, f"culsh_pslsh_query_{sfx}")(self.h, ptr(dQ), nq, ih, batch_size, C.byref(ch)))
        return self.candidates_arrays(ch)

    def pslsh_fit_query(self, X, T, H, w, seed=42, P=None, b=None):
        n, d = X.shape
        sfx = "f32" if X.dtype == np.float32 else "f64"
        dX = dev(X)
        Pc = None if P is None else np.ascontiguousarray(P, dtype=X.dtype)
        bc = None if b is None else np.ascontiguousarray(b, dtype=X.dtype)
        ch = C.c_void_p()
        L.check(getattr(self.lib, f"culsh_pslsh_fit_query_{sfx}")(self.h, ptr(dX), n, d, T, H, w, seed, hp(Pc), hp(bc), C.byref(ch)))
        return self.candidates_arrays(ch)

    def minhash_fit(self, indices, indptr, d, T, H, seed=42, A=None, B=None):
        n = len(indptr) - 1
        di, dp = dev(indices.astype(np.int32)), dev(indptr.astype(np.int32))
        Ac = None if A is None else np.ascontiguousarray(A, dtype=np.uint32)
        Bc = None if B is None else np.ascontiguousarray(B, dtype=np.uint32)
        ih = C.c_void_p()
        L.check(self.lib.culsh_minhash_fit(self.h, ptr(di), ptr(dp), n, d, T, H, seed, hp(Ac), hp(Bc), C.byref(ih)))
        return ih

    def minhash_query(self, indices, indptr, ih):
        nq = len(indptr) - 1
        di, dp = dev(indices.astype(np.int32)), dev(indptr.astype(np.int32))
        ch = C.c_void_p()
        L.check(self.lib.culsh_minhash_query(self.h, ptr(di), ptr(dp), nq, ih, C.byref(ch)))
        return self.candidates_arrays(ch)

    def minhash_fit_query(self, indices, indptr, d, T, H, seed=42, A=None, B=None):
        n = len(indptr) - 1
        di, dp = dev(indices.astype(np.int32)), dev(indptr.astype(np.int32))
        Ac = None if A is None else np.ascontiguousarray(A, dtype=np.uint32)
        Bc = None if B is None else np.ascontiguousarray(B, dtype=np.uint32)
        ch = C.c_void_p()
        L.check(self.lib.culsh_minhash_fit_query(self.h, ptr(di), ptr(dp), n, d, T, H, seed, hp(Ac), hp(Bc), C.byref(ch)))
        return self.candidates_arrays(ch)
