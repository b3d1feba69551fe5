"""
CPU restatement (numpy) of cuLSH's fit/query hot path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke()
and the cpu_baseline leg of bench.py may import it; the shipped package never does.

Every function cites the reference file:line it restates (paths relative to the
reference checkout).  Arithmetic that the reference delegates to closed-source
libraries is restated from the published definition:

  * cuBLAS S/DGEMM (rplsh/hash.cuh:110-117, pslsh/hash.cuh:123-130): X @ P.T.  The
    summation order is unspecified, so hash bits whose projection lies within
    1e-5 relative of the decision boundary are implementation-defined; the
    helpers `rplsh_margin` / `pslsh_margin` return the per-bit margin so tests
    can exclude exactly that band.
  * cuRAND XORWOW (rplsh/hash.cuh:61-69, pslsh/hash.cuh:63-79,
    minhash/hash.cuh:44-49): no reference test pins the generated values
    ("parity unpinned" for the raw random stream).  `generate_*` below are this
    build's own documented counter-based generator; parity of everything
    downstream is defined given identical P / b / A / B.
  * CUB radix sort / scan / select / segmented sort / segmented reduce
    (core/fit.cuh:260-326, core/query.cuh:330-465): stable sort, exact integer
    sums and order-preserving compaction - restated with numpy's stable sorts.

Pinning (see tests/test_oracle.py): every function here is checked against an
independent brute-force model (dict-of-lists LSH as in python/tests/ref_lsh.py,
Python big-int MinHash, hand-built known-answer cases) or a mathematical
invariant, never against a retyped copy of itself.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import numpy as np

MINHASH_PRIME = 4294967291  # minhash/hash.cuh:17 (largest 32-bit prime, 2**32 - 5)
# The prime is a parameter of the functions below; the reference's is the default.  The library also
# takes 2**31 - 1, for which there is no reference code: that case is pinned by big-integer arithmetic
# only (tests/test_oracle.py).
MINHASH_PRIME_MERSENNE = 2147483647

_M64 = (1 << 64) - 1
_GOLD = 0x9E3779B97F4A7C15

# Stream ids of the seeded generator (one independent stream per parameter array).
STREAM_PROJECTION = 1
STREAM_BIAS = 2
STREAM_HASH_A = 3
STREAM_HASH_B = 4


# --------------------------------------------------------------------------------------
# Seeded parameter generator (this build's own; replaces cuRAND XORWOW, see header)
# --------------------------------------------------------------------------------------
def _splitmix64(x: np.ndarray) -> np.ndarray:
    """splitmix64 output function on uint64 arrays (wrapping arithmetic)."""
    with np.errstate(over="ignore"):
        z = x + np.uint64(_GOLD)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def _splitmix64_int(x: int) -> int:
    z = (x + _GOLD) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def stream_key(seed: int, stream: int) -> int:
    """Key of stream `stream` for `seed`: sm64(sm64(seed) ^ sm64(stream))."""
    return _splitmix64_int(_splitmix64_int(seed & _M64) ^ _splitmix64_int(stream))


def raw_u64(seed: int, stream: int, n: int) -> np.ndarray:
    """r[i] = sm64(key + i), i in [0, n)."""
    key = np.uint64(stream_key(seed, stream))
    with np.errstate(over="ignore"):
        return _splitmix64(key + np.arange(n, dtype=np.uint64))


def normal_f64_exact(seed: int, stream: int, n: int) -> np.ndarray:
    """Box-Muller normals through Python's libm (bit-identical to a C++ <cmath> build).

    z[i] = sqrt(-2 ln u1) * cos(2 pi u2), u1 = ((r[2i] >> 11) + 1) * 2^-53 in (0,1],
    u2 = (r[2i+1] >> 11) * 2^-53 in [0,1).
    """
    r = raw_u64(seed, stream, 2 * n)
    out = np.empty(n, dtype=np.float64)
    two_pi = 6.283185307179586476925286766559
    for i in range(n):
        u1 = ((int(r[2 * i]) >> 11) + 1) * (1.0 / 9007199254740992.0)
        u2 = (int(r[2 * i + 1]) >> 11) * (1.0 / 9007199254740992.0)
        out[i] = math.sqrt(-2.0 * math.log(u1)) * math.cos(two_pi * u2)
    return out


def normal_f64(seed: int, stream: int, n: int) -> np.ndarray:
    """Vectorised version of `normal_f64_exact` (numpy libm: may differ in the last ulp)."""
    r = raw_u64(seed, stream, 2 * n)
    u1 = ((r[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
    u2 = (r[1::2] >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586476925286766559 * u2)


def generate_random_projections(seed: int, n_rows: int, d: int, dtype=np.float32) -> np.ndarray:
    """P ~ N(0,1), shape (n_rows, d) row-major (role of rplsh/hash.cuh:58-78)."""
    return normal_f64(seed, STREAM_PROJECTION, n_rows * d).astype(dtype).reshape(n_rows, d)


def generate_random_projections_biases(seed: int, n_rows: int, d: int, w: int, dtype=np.float32):
    """P ~ N(0,1)/w and b ~ U(0,1] (role of pslsh/hash.cuh:59-89; P is divided by the
    integer window in the array's own precision, b is NOT scaled)."""
    P = normal_f64(seed, STREAM_PROJECTION, n_rows * d).astype(dtype).reshape(n_rows, d)
    P = (P / dtype(w)).astype(dtype)
    r = raw_u64(seed, STREAM_BIAS, n_rows)
    b = ((r >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
    return P, b.astype(dtype)


def normalize_hash_integers(raw_a: np.ndarray, raw_b: np.ndarray, prime: int = MINHASH_PRIME):
    """A = raw mod (p-1) + 1 in [1,p-1], B = raw mod p (minhash/hash.cuh:26-32)."""
    A = (raw_a.astype(np.uint64) % np.uint64(prime - 1)) + np.uint64(1)
    B = raw_b.astype(np.uint64) % np.uint64(prime)
    return A.astype(np.uint32), B.astype(np.uint32)


def generate_hash_integers(seed: int, n: int, prime: int = MINHASH_PRIME):
    """Seeded uint32 A, B, normalised as minhash/hash.cuh:42-54."""
    raw_a = (raw_u64(seed, STREAM_HASH_A, n) >> np.uint64(32)).astype(np.uint32)
    raw_b = (raw_u64(seed, STREAM_HASH_B, n) >> np.uint64(32)).astype(np.uint32)
    return normalize_hash_integers(raw_a, raw_b, prime)


# --------------------------------------------------------------------------------------
# Hashing: signatures in the reference's table-major layout X_sig[T][n][H]
# --------------------------------------------------------------------------------------
def _table_major(H_row_major: np.ndarray, T: int, H: int) -> np.ndarray:
    """[n][T*H] -> [T][n][H]  (index arithmetic of rplsh/hash.cuh:35-44)."""
    n = H_row_major.shape[0]
    return np.ascontiguousarray(H_row_major.reshape(n, T, H).transpose(1, 0, 2))


def rplsh_project(X: np.ndarray, P: np.ndarray) -> np.ndarray:
    """X @ P.T accumulated in float64 (exact-summation stand-in for the GEMM at
    rplsh/hash.cuh:110-117)."""
    return X.astype(np.float64) @ P.astype(np.float64).T


def rplsh_sign_bits(X_hash: np.ndarray) -> np.ndarray:
    """sig = (float_bits(x) >> 31) ^ 1: 1 iff the sign bit is clear, so +0.0 -> 1 and
    -0.0 -> 0; a double is narrowed to float first, which keeps its sign
    (rplsh/hash.cuh:47)."""
    return (~np.signbit(X_hash)).astype(np.uint8)


def rplsh_hash(X: np.ndarray, P: np.ndarray, T: int, H: int) -> np.ndarray:
    """uint8 X_sig[T][n][H] (rplsh/hash.cuh:92-129)."""
    return _table_major(rplsh_sign_bits(rplsh_project(X, P)), T, H)


def rplsh_margin(X: np.ndarray, P: np.ndarray, T: int, H: int) -> np.ndarray:
    """|proj| / sum_i |x_i p_i| in table-major layout: a bit is implementation-defined
    where this is <= 1e-5 (band of the unspecified GEMM summation order)."""
    Xd, Pd = X.astype(np.float64), P.astype(np.float64)
    num = np.abs(Xd @ Pd.T)
    den = np.abs(Xd) @ np.abs(Pd).T
    with np.errstate(divide="ignore", invalid="ignore"):
        m = np.where(den > 0, num / den, np.inf)
    return _table_major(m, T, H)


def pslsh_hash(X: np.ndarray, P: np.ndarray, b: np.ndarray, T: int, H: int) -> np.ndarray:
    """int32 X_sig[T][n][H] = floor(X @ P.T + b); P already divided by the window and
    b in (0,1] (pslsh/hash.cuh:25-47, 104-142)."""
    proj = X.astype(np.float64) @ P.astype(np.float64).T + b.astype(np.float64)[None, :]
    return _table_major(np.floor(proj).astype(np.int32), T, H)


def pslsh_margin(X: np.ndarray, P: np.ndarray, b: np.ndarray, T: int, H: int) -> np.ndarray:
    """Distance of (X @ P.T + b) to the nearest integer, relative to
    sum_i |x_i p_i| + |b|: the floor is implementation-defined where this is <= 1e-5."""
    Xd, Pd, bd = X.astype(np.float64), P.astype(np.float64), b.astype(np.float64)
    v = Xd @ Pd.T + bd[None, :]
    dist = np.abs(v - np.rint(v))
    den = np.abs(Xd) @ np.abs(Pd).T + np.abs(bd)[None, :]
    with np.errstate(divide="ignore", invalid="ignore"):
        m = np.where(den > 0, dist / den, np.inf)
    return _table_major(m, T, H)


def minhash_hash(indices: np.ndarray, indptr: np.ndarray, A: np.ndarray, B: np.ndarray,
                 T: int, H: int, prime: int = MINHASH_PRIME) -> np.ndarray:
    """uint32 X_sig[T][n][H] = min_j ((uint64)A*idx_j + B) mod p; empty row -> 0xFFFFFFFF;
    CSR values are ignored (minhash/hash.cuh:69-128)."""
    n = len(indptr) - 1
    TH = T * H
    A64 = A.astype(np.uint64)[:TH]
    B64 = B.astype(np.uint64)[:TH]
    sig = np.full((n, TH), 0xFFFFFFFF, dtype=np.uint32)
    idx64 = indices.astype(np.uint32).astype(np.uint64)  # static_cast<uint32_t>(X_indices[j])
    counts = np.diff(indptr)
    nonempty = np.flatnonzero(counts > 0)
    if len(nonempty) and len(idx64):
        # (A < 2^32) * (idx < 2^32) + (B < 2^32) < 2^64: no wrap in uint64
        for h in range(TH):
            hashed = (A64[h] * idx64 + B64[h]) % np.uint64(prime)
            mins = np.minimum.reduceat(hashed, indptr[nonempty].astype(np.int64))
            sig[nonempty, h] = mins.astype(np.uint32)
    return _table_major(sig, T, H)


# --------------------------------------------------------------------------------------
# Index build (core/fit.cuh)
# --------------------------------------------------------------------------------------
@dataclass
class Index:
    """Host mirror of core::Index (core/index.cuh:12-40)."""
    all_candidate_indices: np.ndarray      # int32 [n_total_candidates]
    all_bucket_signatures: np.ndarray      # uint8 [n_total_buckets * sig_nbytes]
    bucket_candidate_offsets: np.ndarray   # int32 [n_total_buckets + 1]
    table_bucket_offsets: np.ndarray       # int32 [n_hash_tables + 1]
    n_total_candidates: int
    n_total_buckets: int
    n_hash_tables: int
    n_hashes: int
    sig_nbytes: int
    item_to_bucket: Optional[np.ndarray] = None  # int32 [n * T], row-major (row, table)


def _sig_bytes(X_sig: np.ndarray) -> np.ndarray:
    """View a [T][n][...] signature array as opaque bytes [T][n][sig_nbytes] in memory
    order (signatures are opaque fixed-width bytes, core/fit.cuh:214-215)."""
    T, n = X_sig.shape[0], X_sig.shape[1]
    return np.ascontiguousarray(X_sig).view(np.uint8).reshape(T, n, -1)


def _byte_lex_order(sig_tn: np.ndarray) -> np.ndarray:
    """Stable argsort of rows of a [n][S] uint8 matrix, bytes compared unsigned from
    byte 0 (most significant) to byte S-1: the result of the LSD passes over bytes
    S-1..0 starting from the identity permutation (core/fit.cuh:254-272)."""
    n, S = sig_tn.shape
    pad = (-S) % 8
    if pad:
        sig_tn = np.concatenate([sig_tn, np.zeros((n, pad), np.uint8)], axis=1)
    words = np.ascontiguousarray(sig_tn).view(">u8")  # [n][ceil(S/8)], big-endian = byte-lex
    keys = [np.arange(n)] + [words[:, c] for c in range(words.shape[1] - 1, -1, -1)]
    return np.lexsort(keys)  # last key is the primary one


def fit_index(X_sig: np.ndarray, n_hashes: int, with_item_to_bucket: bool = False) -> Index:
    """core::detail::fit_index (core/fit.cuh:222-374).

    Items (table, row) are ordered by (table, signature bytes, row); a bucket is a run
    of equal (table, signature).  Offsets carry terminators: table_bucket_offsets[T] =
    n_total_buckets and bucket_candidate_offsets[n_total_buckets] = n_items
    (core/fit.cuh:351-357)."""
    sig = _sig_bytes(X_sig)
    T, n, S = sig.shape
    cand = np.empty(T * n, dtype=np.int32)
    bucket_sigs, bucket_offs = [], []
    table_offs = np.zeros(T + 1, dtype=np.int32)
    item_to_bucket = np.empty(n * T, dtype=np.int32) if with_item_to_bucket else None
    n_buckets = 0
    for t in range(T):
        order = _byte_lex_order(sig[t])
        s_sorted = sig[t][order]
        cand[t * n:(t + 1) * n] = order
        if n:
            head = np.ones(n, dtype=bool)
            head[1:] = np.any(s_sorted[1:] != s_sorted[:-1], axis=1)   # fit.cuh:126-143
        else:
            head = np.zeros(0, dtype=bool)
        heads = np.flatnonzero(head)
        table_offs[t] = n_buckets
        bucket_offs.append(heads.astype(np.int64) + t * n)              # fit.cuh:190-191
        bucket_sigs.append(s_sorted[heads])                             # fit.cuh:193-205
        if with_item_to_bucket:
            bucket_of_pos = n_buckets + np.cumsum(head) - 1             # fit.cuh:180-185
            item_to_bucket[order.astype(np.int64) * T + t] = bucket_of_pos
        n_buckets += len(heads)
    table_offs[T] = n_buckets
    bco = np.concatenate(bucket_offs + [np.array([T * n], dtype=np.int64)]).astype(np.int32)
    sigs = (np.concatenate(bucket_sigs, axis=0) if n_buckets else np.zeros((0, S), np.uint8))
    return Index(cand, np.ascontiguousarray(sigs).reshape(-1), bco, table_offs,
                 T * n, n_buckets, T, n_hashes, S, item_to_bucket)


# --------------------------------------------------------------------------------------
# Query (core/query.cuh)
# --------------------------------------------------------------------------------------
@dataclass
class Candidates:
    """Host mirror of core::Candidates (core/candidates.cuh:14-40)."""
    query_candidate_indices: np.ndarray   # int32 [n_total_candidates]
    query_candidate_counts: np.ndarray    # uint64 [n_queries]
    query_candidate_offsets: np.ndarray   # uint64 [n_queries + 1]
    n_queries: int
    n_total_candidates: int


def find_matching_buckets(Q_sig: np.ndarray, index: Index) -> np.ndarray:
    """matched[q*T + t] = bucket id whose signature equals Q_sig[t][q], else -1; binary
    search with unsigned byte-wise compare (core/query.cuh:31-101)."""
    qs = _sig_bytes(Q_sig)
    T, nq, S = qs.shape
    assert S == index.sig_nbytes and T == index.n_hash_tables
    bsig = index.all_bucket_signatures.reshape(-1, S)
    matched = np.full(nq * T, -1, dtype=np.int32)
    for t in range(T):
        lo0, hi0 = int(index.table_bucket_offsets[t]), int(index.table_bucket_offsets[t + 1])
        for q in range(nq):
            key = qs[t, q].tobytes()
            lo, hi = lo0, hi0 - 1
            while lo <= hi:
                mid = lo + (hi - lo) // 2
                m = bsig[mid].tobytes()
                if key == m:
                    matched[q * T + t] = mid
                    break
                if key < m:      # Python bytes compare = unsigned lexicographic
                    hi = mid - 1
                else:
                    lo = mid + 1
    return matched


def find_matching_buckets_fast(Q_sig: np.ndarray, index: Index) -> np.ndarray:
    """Same result as `find_matching_buckets` via a per-table dict (for larger sizes)."""
    qs = _sig_bytes(Q_sig)
    T, nq, S = qs.shape
    bsig = index.all_bucket_signatures.reshape(-1, S)
    matched = np.full(nq * T, -1, dtype=np.int32)
    for t in range(T):
        lo, hi = int(index.table_bucket_offsets[t]), int(index.table_bucket_offsets[t + 1])
        table = {bsig[i].tobytes(): i for i in range(lo, hi)}
        for q in range(nq):
            matched[q * T + t] = table.get(qs[t, q].tobytes(), -1)
    return matched


def query_from_matched_buckets(matched: np.ndarray, n_queries: int, index: Index) -> Candidates:
    """core::detail::query_from_matched_buckets (core/query.cuh:290-478): gather the
    spans of the matched buckets table by table, sort each query's segment ascending,
    drop duplicates; counts/offsets are uint64 with offsets[n_queries] = total."""
    T = index.n_hash_tables
    bco = index.bucket_candidate_offsets
    out, counts = [], np.zeros(n_queries, dtype=np.uint64)
    for q in range(n_queries):
        parts = []
        for t in range(T):
            bkt = int(matched[q * T + t])
            if bkt >= 0:
                parts.append(index.all_candidate_indices[int(bco[bkt]):int(bco[bkt + 1])])
        if parts:
            u = np.unique(np.concatenate(parts))          # ascending + unique
            out.append(u.astype(np.int32))
            counts[q] = len(u)
    offsets = np.zeros(n_queries + 1, dtype=np.uint64)
    offsets[1:] = np.cumsum(counts, dtype=np.uint64)
    idx = np.concatenate(out).astype(np.int32) if out else np.zeros(0, dtype=np.int32)
    return Candidates(idx, counts, offsets, n_queries, int(offsets[-1]))


def query_index(Q_sig: np.ndarray, index: Index, fast: bool = True) -> Candidates:
    """core::detail::query_index (core/query.cuh:490-522)."""
    f = find_matching_buckets_fast if fast else find_matching_buckets
    nq = Q_sig.shape[1]
    return query_from_matched_buckets(f(Q_sig, index), nq, index)


def fit_query(X_sig: np.ndarray, n_hashes: int) -> Candidates:
    """core::detail::fit_query (core/fit_query.cuh:30-55): build the index recording
    (row, table) -> bucket, then run the query tail with n_queries = n_samples."""
    index = fit_index(X_sig, n_hashes, with_item_to_bucket=True)
    return query_from_matched_buckets(index.item_to_bucket, X_sig.shape[1], index)


def merge(a: Optional[Candidates], b: Candidates) -> Candidates:
    """Candidates::merge (core/candidates.cuh:139-197): concatenate indices and counts,
    append b's offsets[1:] shifted by a's total."""
    if a is None:
        return b
    idx = np.concatenate([a.query_candidate_indices, b.query_candidate_indices])
    cnt = np.concatenate([a.query_candidate_counts, b.query_candidate_counts])
    off = np.concatenate([a.query_candidate_offsets,
                          b.query_candidate_offsets[1:] + np.uint64(a.n_total_candidates)])
    return Candidates(idx, cnt, off, a.n_queries + b.n_queries,
                      a.n_total_candidates + b.n_total_candidates)


def query_batched(hash_fn, Q, index: Index, batch_size: int) -> Candidates:
    """rplsh::query_batched (rplsh/rplsh.cu:188-206): batch_size <= 0 or >= n_queries is
    the unbatched query; otherwise consecutive row blocks are queried and merged."""
    nq = Q.shape[0]
    if batch_size <= 0 or batch_size >= nq:
        return query_index(hash_fn(Q), index)
    result = None
    for start in range(0, nq, batch_size):
        result = merge(result, query_index(hash_fn(Q[start:start + batch_size]), index))
    return result
