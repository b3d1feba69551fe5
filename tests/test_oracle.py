"""
Pins the CPU oracle (oracle/culsh_oracle.py and oracle/culsh_oracle.c).

The reference ships no golden vectors for this path (its tests are statistical or
self-consistency checks), so each oracle function is pinned against an independent
formulation that a plausible mistake would break:

  * index build / query: a dict-of-lists LSH (the semantic model of the reference's
    python/tests/ref_lsh.py:56-95,139-176) plus Python `sorted()` over bytes objects
    for the bucket order - no lexsort, no radix passes;
  * a hand-computed known-answer case;
  * MinHash: Python big-int arithmetic;
  * sign / floor rules: constructed +0/-0 and boundary inputs, and the reference test
    model's `X @ H.T > 0` / `floor((X @ P.T + b) / w)` (ref_lsh.py:195-197, :275-279);
  * the reference's exact invariants: fit_query == fit+query (test_rplsh.py:145-174),
    batched == unbatched (test_rplsh.py:177-209);
  * the two restatements (numpy, C) against each other.
"""

import math
from collections import defaultdict

import numpy as np
import pytest

from oracle import culsh_oracle as o


# ---------------------------------------------------------------- brute-force models
def brute_index(sig):
    """dict-of-lists index per table; bucket order = sorted(bytes)."""
    sigb = np.ascontiguousarray(sig).view(np.uint8).reshape(sig.shape[0], sig.shape[1], -1)
    T, n, S = sigb.shape
    tables = []
    for t in range(T):
        d = defaultdict(list)
        for i in range(n):
            d[sigb[t, i].tobytes()].append(i)
        tables.append(d)
    cand, bsig, boff, toff = [], [], [], []
    for t in range(T):
        toff.append(len(boff))
        for key in sorted(tables[t].keys()):
            boff.append(len(cand))
            bsig.append(np.frombuffer(key, dtype=np.uint8))
            cand.extend(tables[t][key])
    toff.append(len(boff))
    boff.append(len(cand))
    return tables, (np.array(cand, np.int32),
                    np.concatenate(bsig) if bsig else np.zeros(0, np.uint8),
                    np.array(boff, np.int32), np.array(toff, np.int32))


def brute_query(tables, qsig):
    qb = np.ascontiguousarray(qsig).view(np.uint8).reshape(qsig.shape[0], qsig.shape[1], -1)
    T, nq, _ = qb.shape
    res = []
    for q in range(nq):
        s = set()
        for t in range(T):
            s.update(tables[t].get(qb[t, q].tobytes(), []))
        res.append(sorted(s))
    return res


def assert_index_equal(ix, expected):
    cand, bsig, boff, toff = expected
    np.testing.assert_array_equal(ix.all_candidate_indices, cand)
    np.testing.assert_array_equal(ix.all_bucket_signatures, bsig)
    np.testing.assert_array_equal(ix.bucket_candidate_offsets, boff)
    np.testing.assert_array_equal(ix.table_bucket_offsets, toff)
    assert ix.n_total_buckets == len(boff) - 1
    assert ix.n_total_candidates == len(cand)
    assert ix.all_candidate_indices.dtype == np.int32
    assert ix.bucket_candidate_offsets.dtype == np.int32
    assert ix.table_bucket_offsets.dtype == np.int32
    assert ix.all_bucket_signatures.dtype == np.uint8


def assert_candidates_equal(c, lists):
    assert c.query_candidate_indices.dtype == np.int32
    assert c.query_candidate_counts.dtype == np.uint64
    assert c.query_candidate_offsets.dtype == np.uint64
    assert c.n_queries == len(lists)
    assert int(c.query_candidate_offsets[0]) == 0
    np.testing.assert_array_equal(c.query_candidate_counts, [len(x) for x in lists])
    np.testing.assert_array_equal(np.diff(c.query_candidate_offsets.astype(np.int64)),
                                  [len(x) for x in lists])
    assert int(c.query_candidate_offsets[-1]) == c.n_total_candidates == sum(map(len, lists))
    flat = [v for x in lists for v in x]
    np.testing.assert_array_equal(c.query_candidate_indices, np.array(flat, dtype=np.int32))


def random_sigs(rng, T, n, H, kind):
    if kind == "rplsh":
        return rng.integers(0, 2, size=(T, n, H), dtype=np.uint8)
    if kind == "pslsh":     # small signed ints: exercises the little-endian byte order
        return rng.integers(-3, 4, size=(T, n, H)).astype(np.int32)
    if kind == "minhash":   # wide unsigned values incl. ones that differ only in high bytes
        v = rng.integers(0, 6, size=(T, n, H)).astype(np.uint32)
        return (v * np.uint32(0x01000193)) ^ np.uint32(0x80000001)
    raise ValueError(kind)


# ---------------------------------------------------------------- index build + query
@pytest.mark.parametrize("kind", ["rplsh", "pslsh", "minhash"])
@pytest.mark.parametrize("T,n,H", [(1, 1, 1), (3, 50, 2), (4, 200, 3), (2, 64, 8)])
def test_fit_index_matches_dict_model(kind, T, n, H, c_oracle):
    rng = np.random.default_rng(7 + T * 1000 + n)
    sig = random_sigs(rng, T, n, H, kind)
    _, expected = brute_index(sig)
    assert_index_equal(o.fit_index(sig, H), expected)
    assert_index_equal(c_oracle.fit_index(sig, H), expected)


def test_fit_index_known_answer():
    """Hand-computed: T=2, n=4, int32 signatures of one hash each.
    Table 0 values [1, -1, 256, 1]: little-endian bytes 01000000, ffffffff, 00010000,
    01000000 -> byte order 256 (00..) < 1 (01..) < -1 (ff..): buckets {2}, {0,3}, {1}.
    Table 1 values [0, 0, 0, 0]: one bucket {0,1,2,3}."""
    sig = np.array([[[1], [-1], [256], [1]], [[0], [0], [0], [0]]], dtype=np.int32)
    ix = o.fit_index(sig, 1, with_item_to_bucket=True)
    np.testing.assert_array_equal(ix.all_candidate_indices, [2, 0, 3, 1, 0, 1, 2, 3])
    np.testing.assert_array_equal(ix.bucket_candidate_offsets, [0, 1, 3, 4, 8])
    np.testing.assert_array_equal(ix.table_bucket_offsets, [0, 3, 4])
    np.testing.assert_array_equal(
        ix.all_bucket_signatures.reshape(-1, 4),
        [[0, 1, 0, 0], [1, 0, 0, 0], [255, 255, 255, 255], [0, 0, 0, 0]])
    # item_to_bucket[row * T + table]
    np.testing.assert_array_equal(ix.item_to_bucket, [1, 3, 2, 3, 0, 3, 1, 3])
    assert (ix.n_total_buckets, ix.n_total_candidates, ix.sig_nbytes) == (4, 8, 4)


def test_fit_index_invariants(c_oracle):
    rng = np.random.default_rng(11)
    T, n, H = 5, 3000, 6
    sig = random_sigs(rng, T, n, H, "rplsh")
    for ix in (o.fit_index(sig, H), c_oracle.fit_index(sig, H)):
        S = ix.sig_nbytes
        assert S == H and ix.table_bucket_offsets[T] == ix.n_total_buckets
        assert ix.bucket_candidate_offsets[ix.n_total_buckets] == T * n
        for t in range(T):
            blk = ix.all_candidate_indices[t * n:(t + 1) * n]
            np.testing.assert_array_equal(np.sort(blk), np.arange(n))   # permutation per table
            lo, hi = ix.table_bucket_offsets[t], ix.table_bucket_offsets[t + 1]
            keys = [ix.all_bucket_signatures[b * S:(b + 1) * S].tobytes() for b in range(lo, hi)]
            assert keys == sorted(set(keys))                            # strictly increasing
            for b in range(lo, hi):
                span = ix.all_candidate_indices[
                    ix.bucket_candidate_offsets[b]:ix.bucket_candidate_offsets[b + 1]]
                assert np.all(np.diff(span) > 0)                        # rows ascending
                assert np.all(sig[t, span] == sig[t, span[0]])          # same signature


@pytest.mark.parametrize("kind", ["rplsh", "pslsh", "minhash"])
def test_query_matches_set_union_model(kind, c_oracle):
    rng = np.random.default_rng(23)
    T, n, nq, H = 4, 300, 40, 3
    sig = random_sigs(rng, T, n, H, kind)
    qsig = random_sigs(rng, T, nq, H, kind)
    qsig[:, :5] = sig[:, :5]                      # guaranteed hits
    if kind != "rplsh":
        qsig[:, 5] = 77                           # guaranteed miss in every table
    tables, _ = brute_index(sig)
    expected = brute_query(tables, qsig)
    ix = o.fit_index(sig, H)
    assert_candidates_equal(o.query_index(qsig, ix, fast=False), expected)
    assert_candidates_equal(o.query_index(qsig, ix, fast=True), expected)
    cix = c_oracle.fit_index_c(sig, H)
    assert_candidates_equal(c_oracle.query_index_c(qsig, cix), expected)
    # matched bucket ids: the bucket found must carry the query's signature
    m = o.find_matching_buckets(qsig, ix).reshape(nq, T)
    np.testing.assert_array_equal(m, o.find_matching_buckets_fast(qsig, ix).reshape(nq, T))
    qb = np.ascontiguousarray(qsig).view(np.uint8).reshape(T, nq, -1)
    S = ix.sig_nbytes
    for q in range(nq):
        for t in range(T):
            present = qb[t, q].tobytes() in tables[t]
            assert (m[q, t] >= 0) == present
            if present:
                b = m[q, t]
                assert ix.table_bucket_offsets[t] <= b < ix.table_bucket_offsets[t + 1]
                assert ix.all_bucket_signatures[b * S:(b + 1) * S].tobytes() == qb[t, q].tobytes()


def test_query_no_candidates_at_all():
    sig = np.zeros((2, 10, 2), dtype=np.uint8)
    qsig = np.ones((2, 3, 2), dtype=np.uint8)
    c = o.query_index(qsig, o.fit_index(sig, 2))
    assert c.n_total_candidates == 0 and len(c.query_candidate_indices) == 0
    np.testing.assert_array_equal(c.query_candidate_offsets, [0, 0, 0, 0])
    np.testing.assert_array_equal(c.query_candidate_counts, [0, 0, 0])


@pytest.mark.parametrize("kind", ["rplsh", "pslsh", "minhash"])
def test_fit_query_equals_fit_then_query(kind, c_oracle):
    """Reference invariant, python/tests/test_rplsh.py:145-174 (and pslsh/minhash twins)."""
    rng = np.random.default_rng(5)
    T, n, H = 3, 400, 2
    sig = random_sigs(rng, T, n, H, kind)
    a = o.fit_query(sig, H)
    b = o.query_index(sig, o.fit_index(sig, H))
    c = c_oracle.fit_query(sig, H)
    for x in (b, c):
        np.testing.assert_array_equal(a.query_candidate_indices, x.query_candidate_indices)
        np.testing.assert_array_equal(a.query_candidate_offsets, x.query_candidate_offsets)
        np.testing.assert_array_equal(a.query_candidate_counts, x.query_candidate_counts)
    # every row is its own candidate
    for q in range(n):
        s, e = int(a.query_candidate_offsets[q]), int(a.query_candidate_offsets[q + 1])
        assert q in a.query_candidate_indices[s:e]


@pytest.mark.parametrize("batch", [1, 7, 10, 50, 100, 1000, 0, -1])
def test_batched_equals_unbatched(batch):
    """Reference invariant, python/tests/test_rplsh.py:177-209; batch rule rplsh.cu:190-192."""
    rng = np.random.default_rng(9)
    T, H, d, n, nq = 4, 4, 16, 500, 100
    X = rng.standard_normal((n, d)).astype(np.float32)
    Q = rng.standard_normal((nq, d)).astype(np.float32)
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    ix = o.fit_index(o.rplsh_hash(X, P, T, H), H)
    full = o.query_index(o.rplsh_hash(Q, P, T, H), ix)
    got = o.query_batched(lambda q: o.rplsh_hash(q, P, T, H), Q, ix, batch)
    np.testing.assert_array_equal(full.query_candidate_indices, got.query_candidate_indices)
    np.testing.assert_array_equal(full.query_candidate_offsets, got.query_candidate_offsets)
    np.testing.assert_array_equal(full.query_candidate_counts, got.query_candidate_counts)
    assert got.n_queries == nq and got.query_candidate_offsets.dtype == np.uint64


def test_merge_known_answer():
    a = o.Candidates(np.array([1, 2, 5], np.int32), np.array([2, 1], np.uint64),
                     np.array([0, 2, 3], np.uint64), 2, 3)
    b = o.Candidates(np.array([7, 9], np.int32), np.array([0, 2], np.uint64),
                     np.array([0, 0, 2], np.uint64), 2, 2)
    m = o.merge(a, b)
    np.testing.assert_array_equal(m.query_candidate_indices, [1, 2, 5, 7, 9])
    np.testing.assert_array_equal(m.query_candidate_counts, [2, 1, 0, 2])
    np.testing.assert_array_equal(m.query_candidate_offsets, [0, 2, 3, 3, 5])
    assert (m.n_queries, m.n_total_candidates) == (4, 5)
    assert o.merge(None, b) is b


# ---------------------------------------------------------------- hashing
def test_rplsh_sign_rule_zero_cases(c_oracle):
    """+0.0 -> 1, -0.0 -> 0 (rplsh/hash.cuh:47): an all-zero row projects to +0 on every
    hash; x = -1 against p = 0 gives -0.0 in IEEE arithmetic."""
    xh = np.array([[0.0, -0.0, 1e-30, -1e-30, 3.0, -3.0]], dtype=np.float32)
    np.testing.assert_array_equal(o.rplsh_sign_bits(xh), [[1, 0, 1, 0, 1, 0]])
    np.testing.assert_array_equal(o.rplsh_sign_bits(xh.astype(np.float64) * 1e-300),
                                  [[1, 0, 1, 0, 1, 0]])   # subnormal/underflowing doubles
    X = np.zeros((2, 4), dtype=np.float32)
    X[1] = [1, 2, 3, 4]
    P = np.array([[1, 1, 1, 1], [-1, -1, -1, -1], [1, -1, 1, -1]], dtype=np.float32)
    sig = o.rplsh_hash(X, P, 3, 1)          # [T=3][n=2][H=1]
    np.testing.assert_array_equal(sig[:, 0, 0], [1, 1, 1])     # zero row: +0 everywhere
    np.testing.assert_array_equal(sig[:, 1, 0], [1, 0, 0])     # 10, -10, -2
    np.testing.assert_array_equal(c_oracle.rplsh_hash(X, P, 3, 1)[:, 1, 0], [1, 0, 0])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_rplsh_hash_matches_reference_test_model(dtype, c_oracle):
    """ref_lsh.py:195-197 hashes with (X @ H.T > 0); identical away from exact zero, and
    the layout is table-major [T][n][H]."""
    rng = np.random.default_rng(3)
    T, H, n, d = 6, 5, 257, 33
    X = rng.standard_normal((n, d)).astype(dtype)
    P = rng.standard_normal((T * H, d)).astype(dtype)
    model = (X.astype(np.float64) @ P.astype(np.float64).T > 0).astype(np.uint8)
    sig = o.rplsh_hash(X, P, T, H)
    assert sig.shape == (T, n, H) and sig.dtype == np.uint8
    for t in range(T):
        np.testing.assert_array_equal(sig[t], model[:, t * H:(t + 1) * H])
    safe = o.rplsh_margin(X, P, T, H) > 1e-5
    csig = c_oracle.rplsh_hash(X, P, T, H)
    np.testing.assert_array_equal(csig[safe], sig[safe])
    assert safe.mean() > 0.999


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (7, 3, 2, 5), (1003, 37, 5, 7), (258, 128, 32, 16)])
def test_blocked_cpu_projection_equals_the_plain_one(shape, c_oracle):
    """The blocked projection that the CPU baseline times keeps every output's summation order, so it
    must agree with the plain loop bit for bit: on random data, on rows and columns that do not fill a
    block, and on the signed zeros of all-zero rows and all-zero hash vectors."""
    n, d, T, H = shape
    rng = np.random.default_rng(n + d)
    X = rng.standard_normal((n, d)).astype(np.float32)
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    X[0] = 0.0
    P[-1] = 0.0
    X[-1] = -np.abs(X[-1])          # x < 0 against p = 0 gives -0.0
    plain = c_oracle.rplsh_hash(X, P, T, H)
    np.testing.assert_array_equal(c_oracle.rplsh_hash(X, P, T, H, blocked=True), plain)
    np.testing.assert_array_equal(plain[:, 0, :], 1)      # the zero row: +0.0 everywhere


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pslsh_hash_matches_reference_test_model(dtype, c_oracle):
    """ref_lsh.py:275-279: floor((X @ P.T + b) / w) with b ~ U[0,w); the reference core
    stores P/w and b/w in (0,1] (pslsh/hash.cuh:71-86), the same family."""
    rng = np.random.default_rng(4)
    T, H, n, d, w = 4, 3, 301, 20, 4
    X = rng.standard_normal((n, d)).astype(dtype)
    P0 = rng.standard_normal((T * H, d)).astype(dtype)
    b0 = rng.uniform(0, w, size=T * H).astype(dtype)
    model = np.floor((X.astype(np.float64) @ P0.astype(np.float64).T + b0) / w).astype(np.int32)
    P, b = (P0 / dtype(w)).astype(dtype), (b0 / dtype(w)).astype(dtype)
    sig = o.pslsh_hash(X, P, b, T, H)
    safe = o.pslsh_margin(X, P, b, T, H) > 1e-5
    assert sig.shape == (T, n, H) and sig.dtype == np.int32 and safe.mean() > 0.99
    for t in range(T):
        s = safe[t]
        np.testing.assert_array_equal(sig[t][s], model[:, t * H:(t + 1) * H][s])
    csig = c_oracle.pslsh_hash(X, P, b, T, H)
    np.testing.assert_array_equal(csig[safe], sig[safe])
    assert sig.min() < 0 < sig.max()          # negative floors are exercised


def test_pslsh_floor_known_answer():
    X = np.array([[1.0], [-1.0], [0.0]], dtype=np.float64)
    P = np.array([[0.5], [2.0]], dtype=np.float64)
    b = np.array([0.25, 1.0], dtype=np.float64)
    # row0: 0.75, 3.0 ; row1: -0.25, -1.0 ; row2: 0.25, 1.0
    sig = o.pslsh_hash(X, P, b, 2, 1)
    np.testing.assert_array_equal(sig[:, :, 0], [[0, -1, 0], [3, -1, 1]])


@pytest.mark.parametrize("prime", [4294967291, 2147483647])
def test_minhash_matches_bigint(c_oracle, prime):
    """Both primes the library takes: the reference's 2^32 - 5 (minhash/hash.cuh:17) and 2^31 - 1."""
    rng = np.random.default_rng(8)
    T, H, n, d = 3, 4, 40, 1000
    rows = [np.sort(rng.choice(d, size=rng.integers(0, 12), replace=False)) for _ in range(n)]
    rows[3] = np.array([], dtype=np.int64)                       # empty row
    rows[4] = np.array([d - 1, d - 1, 5])                        # duplicate index is harmless
    rows[5] = np.array([2**31 - 1])                              # largest int32 column id
    indptr = np.concatenate([[0], np.cumsum([len(r) for r in rows])]).astype(np.int32)
    indices = np.concatenate(rows).astype(np.int32)
    A = rng.integers(1, prime, size=T * H, dtype=np.uint64).astype(np.uint32)
    B = rng.integers(0, prime, size=T * H, dtype=np.uint64).astype(np.uint32)
    A[0], B[0] = prime - 1, prime - 1                            # extremes of the ranges
    A[1], B[1] = 0xFFFFFFFF, 0xFFFFFFFF                          # injected parameters need not be normalised
    expected = np.empty((T, n, H), dtype=np.uint32)
    for i, r in enumerate(rows):
        for c in range(T * H):
            vals = [(int(A[c]) * int(x) + int(B[c])) % prime for x in r]
            expected[c // H, i, c % H] = min(vals) if vals else 0xFFFFFFFF
    np.testing.assert_array_equal(o.minhash_hash(indices, indptr, A, B, T, H, prime), expected)
    np.testing.assert_array_equal(c_oracle.minhash_hash(indices, indptr, A, B, T, H, prime), expected)
    if prime == o.MINHASH_PRIME:                                 # the default is the reference's prime
        np.testing.assert_array_equal(o.minhash_hash(indices, indptr, A, B, T, H), expected)
        np.testing.assert_array_equal(c_oracle.minhash_hash(indices, indptr, A, B, T, H), expected)


def test_minhash_jaccard_estimate():
    """Mathematical property: P[minhash equal] = Jaccard similarity."""
    rng = np.random.default_rng(12)
    d = 5000
    a = rng.choice(d, 300, replace=False)
    b = np.concatenate([a[:200], rng.choice(np.setdiff1d(np.arange(d), a), 100, replace=False)])
    jac = len(np.intersect1d(a, b)) / len(np.union1d(a, b))
    indices = np.concatenate([np.sort(a), np.sort(b)]).astype(np.int32)
    indptr = np.array([0, 300, 600], dtype=np.int32)
    A, B = o.generate_hash_integers(99, 4000)
    sig = o.minhash_hash(indices, indptr, A, B, 1, 4000)
    est = np.mean(sig[0, 0] == sig[0, 1])
    assert abs(est - jac) < 0.03


# ---------------------------------------------------------------- seeded generator
def test_generator_exact_and_vectorised_agree():
    ex = o.normal_f64_exact(42, o.STREAM_PROJECTION, 2000)
    vec = o.normal_f64(42, o.STREAM_PROJECTION, 2000)
    np.testing.assert_allclose(vec, ex, rtol=4e-15, atol=1e-300)
    # first element from the definition, with Python ints + math only
    key = o.stream_key(42, o.STREAM_PROJECTION)
    r0 = o._splitmix64_int(key)
    r1 = o._splitmix64_int((key + 1) & ((1 << 64) - 1))
    u1 = ((r0 >> 11) + 1) / 2.0**53
    u2 = (r1 >> 11) / 2.0**53
    assert ex[0] == math.sqrt(-2.0 * math.log(u1)) * math.cos(2 * math.pi * u2)


def test_splitmix64_known_answer():
    """splitmix64 with state 0 emits 0xE220A8397B1DCDAF first (published test vector)."""
    assert o._splitmix64_int(0) == 0xE220A8397B1DCDAF
    assert int(o._splitmix64(np.array([0], dtype=np.uint64))[0]) == 0xE220A8397B1DCDAF


def test_generator_statistics_and_ranges():
    P = o.generate_random_projections(7, 512, 128)
    assert P.shape == (512, 128) and P.dtype == np.float32
    assert abs(P.mean()) < 0.02 and abs(P.std() - 1.0) < 0.02
    assert not np.array_equal(P, o.generate_random_projections(8, 512, 128))
    np.testing.assert_array_equal(P, o.generate_random_projections(7, 512, 128))
    Pw, b = o.generate_random_projections_biases(7, 512, 128, 4)
    np.testing.assert_array_equal(Pw, (P / np.float32(4)).astype(np.float32))
    assert b.min() > 0.0 and b.max() <= 1.0 and abs(b.mean() - 0.5) < 0.05
    A, B = o.generate_hash_integers(7, 4096)
    assert A.dtype == np.uint32 and A.min() >= 1 and int(A.max()) <= o.MINHASH_PRIME - 1
    assert int(B.max()) <= o.MINHASH_PRIME - 1 and not np.array_equal(A, B)
    rawa = np.array([0, o.MINHASH_PRIME - 2, o.MINHASH_PRIME - 1, 2**32 - 1], dtype=np.uint32)
    a2, b2 = o.normalize_hash_integers(rawa, rawa)
    np.testing.assert_array_equal(a2, [1, o.MINHASH_PRIME - 1, 1, 6])   # (2^32-1) mod (p-1) = 5, +1
    np.testing.assert_array_equal(b2, [0, o.MINHASH_PRIME - 2, o.MINHASH_PRIME - 1, 4])


# ---------------------------------------------------------------- end to end vs ref model
def test_end_to_end_rplsh_vs_dict_lsh(c_oracle):
    """Whole path (hash -> fit -> query) against the dict-of-lists LSH of ref_lsh.py."""
    rng = np.random.default_rng(31)
    T, H, n, nq, d = 8, 6, 1000, 60, 24
    X = rng.standard_normal((n, d)).astype(np.float32)
    Q = (X[:nq] + 0.1 * rng.standard_normal((nq, d))).astype(np.float32)
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    hx = (X.astype(np.float64) @ P.astype(np.float64).T > 0).astype(int)
    hq = (Q.astype(np.float64) @ P.astype(np.float64).T > 0).astype(int)
    index = [defaultdict(list) for _ in range(T)]
    for i, s in enumerate(hx):
        for j in range(T):
            index[j][tuple(s[j * H:(j + 1) * H])].append(i)
    expected = []
    for s in hq:
        c = set()
        for j in range(T):
            c.update(index[j].get(tuple(s[j * H:(j + 1) * H]), []))
        expected.append(sorted(c))
    ix = o.fit_index(o.rplsh_hash(X, P, T, H), H)
    assert_candidates_equal(o.query_index(o.rplsh_hash(Q, P, T, H), ix), expected)
    assert sum(map(len, expected)) > nq      # the case is not vacuous
