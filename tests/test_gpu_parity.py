"""
GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle on the
same seeded inputs.

Bar: bucket tables, matched buckets and candidate lists are bit-exact given identical
signatures; MinHash signatures are bit-exact; RPLSH / p-stable hash values may differ
from the float64 oracle only where the projection lies within 1e-5 (relative to
sum |x_i p_i|) of the decision boundary - the band left open by the unspecified
summation order of the reference's GEMM.
"""

import numpy as np
import pytest

from oracle import culsh_oracle as o

pytestmark = pytest.mark.gpu

TOL = 1e-5  # relative width of the implementation-defined band around a hash boundary


@pytest.fixture(scope="module")
def ctx():
    from abi import Ctx

    c = Ctx(0)
    yield c
    c.close()


def _announce(*a):
    print("[case]", *a, flush=True)


def random_sigs(rng, T, n, H, kind):
    if kind == "rplsh":
        return rng.integers(0, 2, size=(T, n, H), dtype=np.uint8)
    if kind == "pslsh":
        return rng.integers(-3, 4, size=(T, n, H)).astype(np.int32)
    if kind == "minhash":
        v = rng.integers(0, 6, size=(T, n, H)).astype(np.uint32)
        return (v * np.uint32(0x01000193)) ^ np.uint32(0x80000001)
    if kind == "bytes3":  # generic opaque signatures whose width is not a multiple of 4
        return rng.integers(0, 3, size=(T, n, 3), dtype=np.uint8) * np.uint8(100)
    raise ValueError(kind)


# ---------------------------------------------------------------- hashing
@pytest.mark.parametrize("n,d,T,H", [
    (1, 8, 1, 1), (257, 100, 8, 8), (1000, 128, 16, 8), (333, 33, 5, 16), (129, 64, 3, 32),
    (200, 40, 4, 20), (150, 128, 2, 40), (300, 36, 3, 64), (4100, 128, 32, 16), (100, 768, 4, 16),
])
def test_rplsh_hash_f32(ctx, n, d, T, H):
    _announce("rplsh_hash_f32", n, d, T, H)
    rng = np.random.default_rng(n * 7 + d)
    X = rng.standard_normal((n, d)).astype(np.float32)
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    got = ctx.rplsh_hash(X, P, T, H)
    exp = o.rplsh_hash(X, P, T, H)
    safe = o.rplsh_margin(X, P, T, H) > TOL
    assert got.shape == exp.shape and safe.mean() > 0.999
    np.testing.assert_array_equal(got[safe], exp[safe])
    assert set(np.unique(got)) <= {0, 1}


def test_rplsh_hash_zero_rule(ctx):
    """+0.0 -> 1 (rplsh/hash.cuh:47): zero rows and zero projections hash to 1; integer
    data with small-integer projections is exact in fp32, so every bit must match."""
    rng = np.random.default_rng(1)
    n, d, T, H = 300, 64, 4, 8
    X = rng.integers(0, 4, size=(n, d)).astype(np.float32)
    X[::7] = 0.0
    P = rng.integers(-2, 3, size=(T * H, d)).astype(np.float32)
    P[5] = 0.0
    got = ctx.rplsh_hash(X, P, T, H)
    proj = X.astype(np.float64) @ P.astype(np.float64).T
    exp = o.rplsh_hash(X, P, T, H)
    np.testing.assert_array_equal(got, exp)
    assert (proj == 0).sum() > n            # exact zeros are exercised
    assert np.all(got[:, ::7, :] == 1)


@pytest.mark.parametrize("n,d,T,H", [(257, 100, 8, 8), (130, 33, 3, 5)])
def test_rplsh_hash_f64(ctx, n, d, T, H):
    _announce("rplsh_hash_f64", n, d, T, H)
    rng = np.random.default_rng(n)
    X = rng.standard_normal((n, d))
    P = rng.standard_normal((T * H, d))
    got = ctx.rplsh_hash(X, P, T, H)
    safe = o.rplsh_margin(X, P, T, H) > 1e-12
    np.testing.assert_array_equal(got[safe], o.rplsh_hash(X, P, T, H)[safe])


@pytest.mark.parametrize("dtype,tol", [(np.float32, TOL), (np.float64, 1e-12)])
@pytest.mark.parametrize("n,d,T,H,w", [(300, 128, 16, 8, 4), (129, 30, 3, 5, 2)])
def test_pslsh_hash(ctx, dtype, tol, n, d, T, H, w):
    _announce("pslsh_hash", dtype.__name__, n, d, T, H, w)
    rng = np.random.default_rng(d)
    X = rng.standard_normal((n, d)).astype(dtype)
    P, b = o.generate_random_projections_biases(5, T * H, d, w, dtype)
    got = ctx.pslsh_hash(X, P, b, T, H)
    exp = o.pslsh_hash(X, P, b, T, H)
    safe = o.pslsh_margin(X, P, b, T, H) > tol
    assert safe.mean() > 0.99 and exp.min() < 0 < exp.max()
    np.testing.assert_array_equal(got[safe], exp[safe])


def make_csr(rng, n, d, mean_nnz, empty_rows=()):
    rows = [np.sort(rng.choice(d, size=min(d, rng.poisson(mean_nnz)), replace=False)) for _ in range(n)]
    for r in empty_rows:
        rows[r] = np.array([], dtype=np.int64)
    indptr = np.concatenate([[0], np.cumsum([len(r) for r in rows])]).astype(np.int32)
    indices = (np.concatenate(rows) if indptr[-1] else np.zeros(0)).astype(np.int32)
    return indices, indptr


@pytest.mark.parametrize("n,d,T,H,nnz", [(1, 10, 1, 1, 3), (500, 5000, 32, 4, 50), (77, 300, 5, 3, 8), (64, 100000, 2, 130, 20)])
def test_minhash_compute_exact(ctx, n, d, T, H, nnz):
    _announce("minhash", n, d, T, H, nnz)
    rng = np.random.default_rng(n + H)
    indices, indptr = make_csr(rng, n, d, nnz, empty_rows=(0,) if n > 1 else ())
    A, B = o.generate_hash_integers(9, T * H)
    A[0], B[0] = o.MINHASH_PRIME - 1, o.MINHASH_PRIME - 1
    got = ctx.minhash_compute(indices, indptr, A, B, T, H)
    np.testing.assert_array_equal(got, o.minhash_hash(indices, indptr, A, B, T, H))


# ---------------------------------------------------------------- index build
@pytest.mark.parametrize("kind", ["rplsh", "pslsh", "minhash", "bytes3"])
@pytest.mark.parametrize("T,n,H", [(1, 1, 1), (3, 50, 2), (4, 5000, 3), (2, 9000, 8), (33, 300, 16)])
def test_core_fit_index(ctx, kind, T, n, H):
    _announce("core_fit_index", kind, T, n, H)
    rng = np.random.default_rng(7 + T * 1000 + n)
    sig = random_sigs(rng, T, n, H, kind)
    ih, itb = ctx.core_fit_index(sig, H, want_item_to_bucket=True)
    from abi import assert_index_matches

    exp = o.fit_index(sig, H, with_item_to_bucket=True)
    assert_index_matches(ctx.index_arrays(ih), exp)
    np.testing.assert_array_equal(itb, exp.item_to_bucket)
    ctx.free_index(ih)


@pytest.mark.parametrize("knob", ["CULSH_SORT_UNCHAINED=1", "CULSH_SORT_SPIN_LIMIT=0"])
def test_core_fit_index_sort_fallbacks(ctx, c_oracle, monkeypatch, knob):
    """The radix sort without the chained scan, and the repeat of a fit after the chained scan
    gave up (forced by allowing no polls; every kernel still runs to its end)."""
    _announce("sort_fallback", knob)
    name, value = knob.split("=")
    monkeypatch.setenv(name, value)
    rng = np.random.default_rng(12)
    T, n, H = 3, 70000, 2          # 18 tiles per table, two radix passes
    sig = rng.integers(0, 256, size=(T, n, H), dtype=np.uint8)
    from abi import Ctx, assert_index_matches

    own = Ctx(0)                    # a give-up switches its context to unchained passes for good
    try:
        ih, _ = own.core_fit_index(sig, H)
        assert_index_matches(own.index_arrays(ih), c_oracle.fit_index_c(sig, H).to_numpy(n))
        own.free_index(ih)
    finally:
        own.close()


def test_fit_after_sort_gives_up_touches_nothing_it_should_not(c_oracle, monkeypatch):
    """A give-up of the chained scan leaves sorted keys and rows incomplete.  The kernels queued behind
    the sort must skip their work on seeing the flag (they would otherwise use stale rows as addresses
    and write more buckets than the arrays sized for sign-bit keys hold), and the repeated fit must
    give the oracle's result: RPLSH fit_query (row -> bucket map, bucket arrays sized by 2^H per table)
    and a MinHash fit whose column sort and item sort both span several tiles."""
    _announce("sort_give_up_fit_query_and_minhash")
    monkeypatch.setenv("CULSH_SORT_SPIN_LIMIT", "0")
    from abi import Ctx, assert_candidates_match, assert_index_matches

    rng = np.random.default_rng(31)
    n, d, T, H = 20000, 32, 4, 8                    # 3 tiles of 8192 one-word keys per table
    X = rng.standard_normal((n, d)).astype(np.float32)
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    own = Ctx(0)                                    # a give-up switches its context to unchained passes for good
    try:
        sig = own.rplsh_hash(X, P, T, H)
        got = own.rplsh_fit_query(X, T, H, seed=1, P=P)
        assert_candidates_match(got, c_oracle.fit_query(sig, H))
    finally:
        own.close()

    n, dcols, T, H = 30000, 20000, 2, 2             # 15-bit rank codes: one key word, 4 tiles; 3 tiles of columns
    indices, indptr = make_csr(rng, n, dcols, 6)
    A, B = o.generate_hash_integers(5, T * H)
    own = Ctx(0)
    try:
        ih = own.minhash_fit(indices, indptr, dcols, T, H, seed=5, A=A, B=B)
        sig = c_oracle.minhash_hash(indices, indptr, A, B, T, H)
        assert_index_matches(own.index_arrays(ih), c_oracle.fit_index_c(sig, H).to_numpy(n))
        own.free_index(ih)
    finally:
        own.close()


def test_more_than_1024_tables_are_refused_up_front(ctx):
    """The query path handles up to 1024 tables (one thread of a workgroup per table), so no index with
    more is ever built: fit, fit_query and load of every family say so before they hash, sort or copy
    anything, instead of handing out an index that no query accepts."""
    import ctypes as C

    from abi import hp
    from culsh_amd import _lib as L

    sig = np.zeros((1025, 4, 1), dtype=np.uint8)
    with pytest.raises(RuntimeError, match="1024"):
        ctx.core_fit_query(sig, 1)
    with pytest.raises(RuntimeError, match="1024"):
        ctx.core_fit_index(sig, 1)
    X = np.zeros((4, 8), dtype=np.float32)
    with pytest.raises(RuntimeError, match="1024"):
        ctx.rplsh_fit_query(X, 1025, 1)
    with pytest.raises(RuntimeError, match="1024"):
        ctx.rplsh_fit(X, 1025, 1)
    with pytest.raises(RuntimeError, match="1024"):
        ctx.pslsh_fit(X, 1025, 1, 4)
    indptr = np.arange(5, dtype=np.int32)
    with pytest.raises(RuntimeError, match="1024"):
        ctx.minhash_fit(np.zeros(4, np.int32), indptr, 8, 1025, 1)
    # a saved index with 1025 tables of one bucket each
    T, n = 1025, 2
    cand = np.tile(np.arange(n, dtype=np.int32), T)
    bsig = np.zeros(T, dtype=np.uint8)
    bco = (np.arange(T + 1) * n).astype(np.int32)
    tbo = np.arange(T + 1, dtype=np.int32)
    ih = C.c_void_p()
    rc = ctx.lib.culsh_index_load(ctx.h, L.KIND_CORE, 0, hp(cand), hp(bsig), hp(bco), hp(tbo), None, None,
                                  T * n, T, T, 1, 1, 0, 0, C.byref(ih))
    assert rc == L.ERR_LIMIT and b"1024" in ctx.lib.culsh_last_error()


def test_core_fit_index_single_bucket_per_table(ctx):
    """All signatures equal: no radix pass runs and rows stay in identity order."""
    sig = np.full((3, 1000, 4), 1, dtype=np.uint8)
    ih, _ = ctx.core_fit_index(sig, 4)
    from abi import assert_index_matches

    assert_index_matches(ctx.index_arrays(ih), o.fit_index(sig, 4))
    ctx.free_index(ih)


def test_core_fit_index_against_c_oracle_larger(ctx, c_oracle):
    rng = np.random.default_rng(99)
    T, n, H = 8, 60000, 12
    sig = rng.integers(0, 2, size=(T, n, H), dtype=np.uint8)
    sig[:, :, :4] = 1       # constant leading bytes
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_index_matches

    assert_index_matches(ctx.index_arrays(ih), c_oracle.fit_index(sig, H))
    ctx.free_index(ih)


# ---------------------------------------------------------------- query
@pytest.mark.parametrize("kind", ["rplsh", "pslsh", "minhash", "bytes3"])
def test_core_query(ctx, kind):
    _announce("core_query", kind)
    rng = np.random.default_rng(23)
    T, n, nq, H = 6, 3000, 200, 3
    sig = random_sigs(rng, T, n, H, kind)
    qsig = random_sigs(rng, T, nq, H, kind)
    qsig[:, :20] = sig[:, :20]
    if kind != "rplsh":
        qsig[:, 20:25] = 77
    ih, _ = ctx.core_fit_index(sig, H)
    exp_ix = o.fit_index(sig, H)
    np.testing.assert_array_equal(ctx.core_find_matching_buckets(qsig, ih),
                                  o.find_matching_buckets_fast(qsig, exp_ix))
    from abi import assert_candidates_match

    got = ctx.core_query_index(qsig, ih)
    assert_candidates_match(got, o.query_index(qsig, exp_ix))
    assert got["counts"].dtype == np.uint64 and got["indices"].dtype == np.int32
    ctx.free_index(ih)


def test_core_query_no_candidates(ctx):
    sig = np.zeros((2, 100, 2), dtype=np.uint8)
    qsig = np.ones((2, 7, 2), dtype=np.uint8)
    ih, _ = ctx.core_fit_index(sig, 2)
    got = ctx.core_query_index(qsig, ih)
    assert got["n_total_candidates"] == 0 and len(got["indices"]) == 0
    np.testing.assert_array_equal(got["offsets"], np.zeros(8, np.uint64))
    np.testing.assert_array_equal(got["counts"], np.zeros(7, np.uint64))
    ctx.free_index(ih)


def test_core_query_from_matched_with_misses(ctx):
    rng = np.random.default_rng(4)
    T, n, H = 5, 2000, 2
    sig = random_sigs(rng, T, n, H, "pslsh")
    ih, _ = ctx.core_fit_index(sig, H)
    exp_ix = o.fit_index(sig, H)
    nq = 64
    matched = rng.integers(-1, exp_ix.n_total_buckets, size=nq * T).astype(np.int32)
    for t in range(T):  # keep each entry inside its table (or -1)
        col = matched[t::T]
        lo, hi = exp_ix.table_bucket_offsets[t], exp_ix.table_bucket_offsets[t + 1]
        col[col >= 0] = lo + col[col >= 0] % (hi - lo)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_from_matched(matched, nq, ih),
                            o.query_from_matched_buckets(matched, nq, exp_ix))
    # ids beyond the buckets are not followed: same result as with -1 in their place
    beyond = matched.copy()
    beyond[matched < 0] = exp_ix.n_total_buckets + np.arange(int((matched < 0).sum()), dtype=np.int32) * 1000
    assert_candidates_match(ctx.core_query_from_matched(beyond, nq, ih),
                            o.query_from_matched_buckets(matched, nq, exp_ix))
    ctx.free_index(ih)


@pytest.mark.parametrize("n", [40000, 1200000])
def test_core_query_wide_row_range(ctx, c_oracle, n):
    """Row ranges beyond one LDS bitmap pass (2^20 rows) and beyond one word per thread."""
    _announce("wide_row_range", n)
    rng = np.random.default_rng(n)
    T, H, nq = 3, 2, 20
    sig = rng.integers(0, 2, size=(T, n, H), dtype=np.uint8)
    qsig = rng.integers(0, 2, size=(T, nq, H), dtype=np.uint8)
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match, assert_index_matches

    cix = c_oracle.fit_index_c(sig, H)
    assert_index_matches(ctx.index_arrays(ih), cix.to_numpy(n))
    assert_candidates_match(ctx.core_query_index(qsig, ih), c_oracle.query_index_c(qsig, cix))
    ctx.free_index(ih)


def test_core_query_output_sized_from_previous_call(ctx, monkeypatch):
    """A second query call on an index sizes its output from the first call's distinct candidates per query
    and reads the true number back afterwards.  Calls whose queries bring fewer, as many, and far more
    candidates than the call before (the last overflows the guessed size and is redone), then forced
    guesses of one candidate per query and of more than the index holds, and a call without any match."""
    _announce("output_sized_from_previous_call")
    from abi import assert_candidates_match

    rng = np.random.default_rng(61)
    T, n, H = 6, 20000, 2
    sig = rng.integers(0, 30, size=(T, n, H)).astype(np.uint8)
    sig[:, :5000, :] = 7                                   # one bucket of 5000 rows per table
    ih, _ = ctx.core_fit_index(sig, H)
    exp_ix = o.fit_index(sig, H)
    few = rng.integers(8, 30, size=(T, 300, H)).astype(np.uint8)
    many = few.copy()
    many[:, ::2, :] = 7                                    # every other query hits the large bucket in every table
    none = np.full((T, 50, H), 200, np.uint8)
    for qsig in (few, few, many, few, none, few, many[:, :10], many):
        assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, exp_ix))
    # A second index of another shape, queried in turns with the first: the sizes are remembered per
    # index shape, so each keeps its own (the first one's large-bucket queries must not size the
    # second one's output, nor the other way round), and every call matches the oracle.
    T2, n2 = 3, 7000
    sig2 = rng.integers(0, 4, size=(T2, n2, H)).astype(np.uint8)          # ~440 rows per bucket
    ih2, _ = ctx.core_fit_index(sig2, H)
    exp_ix2 = o.fit_index(sig2, H)
    q2 = rng.integers(0, 4, size=(T2, 200, H)).astype(np.uint8)
    for _ in range(3):
        assert_candidates_match(ctx.core_query_index(many, ih), o.query_index(many, exp_ix))
        assert_candidates_match(ctx.core_query_index(q2, ih2), o.query_index(q2, exp_ix2))
        assert_candidates_match(ctx.core_query_index(few, ih), o.query_index(few, exp_ix))
    ctx.free_index(ih2)
    for forced in ("1", "100000000", "0"):
        monkeypatch.setenv("CULSH_QUERY_RAW_GUESS", forced)
        for qsig in (many, none, few):
            assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, exp_ix))
    ctx.free_index(ih)


@pytest.mark.parametrize("top", [0xFFFFFFFF, 0x000FFFFF, 0x00000FFF, 5, 0])
def test_core_lookup_directory_edges(ctx, top):
    """The lookup narrows its binary search through a directory over the leading bits of the keys'
    first words, counted from the highest bit any bucket key has set.  Keys at both ends of the range
    up to `top`, directory cells that are empty, full or shared by many buckets, and query keys below,
    between and beyond the bucket keys (also beyond `top`) must all be found or missed as by the oracle."""
    _announce("lookup_directory_edges", top)
    rng = np.random.default_rng(top % 1000 + 3)
    T, n, nq = 3, 3000, 600

    def as_sig(words):  # opaque 4-byte signatures whose byte order is the key order
        return np.ascontiguousarray(words.astype(">u4")).view(np.uint8).reshape(words.shape + (4,))

    special = np.array([0, 1, top // 2, max(top, 1) - 1, top], dtype=np.uint64)
    words = rng.integers(0, int(top) + 1, size=(T, n), dtype=np.uint64)
    words[:, :400] = words[:, :1] // 2                      # one crowded bucket per table
    words[:, 400:400 + special.size] = special
    words[2, :] = top                                       # a table with a single bucket, at the top
    q = rng.integers(0, min(int(top) * 2 + 2, 1 << 32), size=(T, nq), dtype=np.uint64)
    q[:, :200] = words[:, rng.integers(0, n, 200)]          # exact hits
    q[:, 200:210] = np.array([0, 1, top, min(top + 1, 0xFFFFFFFF), 0xFFFFFFFF, top // 2, 2, 3, 4, 5], dtype=np.uint64)
    q[:, 210:300] = np.minimum(words[:, 1000:1090] + 1, 0xFFFFFFFF)   # just beside a bucket key
    sig, qsig = as_sig(words.astype(np.uint32)), as_sig(q.astype(np.uint32))
    ih, _ = ctx.core_fit_index(sig, 1)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, o.fit_index(sig, 1)))
    ctx.free_index(ih)


@pytest.mark.parametrize("two_pass", [False, True])
def test_core_query_many_bitmap_passes(ctx, monkeypatch, two_pass):
    """A small bitmap (32768 rows per pass) makes a 150k-row index take five passes per query: in the
    single launch every span is cut at the passes' row bounds and the lists are written at raw-count
    spacing, then moved together; passes without any row and queries without candidates are among
    them.  Also through the count / scan / emit launches."""
    _announce("many_bitmap_passes", two_pass)
    monkeypatch.setenv("CULSH_DEDUP_WPT", "1")
    if two_pass:
        monkeypatch.setenv("CULSH_DEDUP_TWO_PASS", "1")
    rng = np.random.default_rng(77)
    T, n, nq, H = 7, 150_000, 1500, 2
    sig = rng.integers(0, 40, size=(T, n, H)).astype(np.uint8)           # ~94 rows per bucket
    sig[:, 40_000:70_000, 0] = 200                                        # rows of the second pass keep to themselves
    qsig = rng.integers(0, 40, size=(T, nq, H)).astype(np.uint8)
    qsig[:, ::9, 0] = 200                                                 # candidates in one pass only
    qsig[:, ::13, :] = 255                                                # no candidates at all
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, o.fit_index(sig, H)))
    ctx.free_index(ih)


def test_core_query_bitmap_passes_long_spans_many_tables(ctx, c_oracle, monkeypatch):
    """Several passes per query with 100 tables (more span cuts than one search round holds, spans
    reloaded per query) and buckets of ~30k rows (every span crosses every row bound, the search
    takes seven rounds), next to buckets of one row and buckets that end exactly at a bound."""
    _announce("bitmap_passes_long_spans_many_tables")
    monkeypatch.setenv("CULSH_DEDUP_WPT", "1")
    rng = np.random.default_rng(78)
    T, n, nq, H = 100, 120_000, 24, 1
    sig = rng.integers(0, 4, size=(T, n, H)).astype(np.uint8)
    sig[:50, :32768, 0] = 9                     # a bucket that is exactly the first pass
    sig[50:, 32768:65536 + 1, 0] = 9            # one that overshoots the second pass by a row
    sig[:, 100_000, 0] = 77                     # single-row buckets in the last pass
    qsig = rng.integers(0, 4, size=(T, nq, H)).astype(np.uint8)
    qsig[:, 3::4, 0] = 9
    qsig[:, 5, 0] = 77
    qsig[:, 6, 0] = 200                         # no candidates
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_index(qsig, ih), c_oracle.query_index_c(qsig, c_oracle.fit_index_c(sig, H)))
    ctx.free_index(ih)


def test_core_query_sparse_passes_at_full_bitmap_size(ctx, c_oracle):
    """1.1M rows: two passes per query over the full-size bitmap (2^20 rows, eight words per lane and
    step).  Passes that hold few rows for their range are read out through the summary of non-zero
    words: buckets of rows that sit in one word, fill words completely, sit at both ends of a word, of
    a lane's 32 words and of a pass, straddle the pass boundary, or are the index's last row; next to a
    query whose passes are dense (read out by the sweep) and one without candidates."""
    _announce("sparse_passes_full_bitmap")
    rng = np.random.default_rng(79)
    T, n, nq, H = 3, 1_100_000, 12, 1
    sig = rng.integers(0, 2, size=(T, n, H)).astype(np.uint8)            # two big buckets per table: dense passes
    edge = 1 << 20
    groups = {
        10: np.arange(edge - 70, edge + 70),                             # across the pass boundary, whole words
        11: np.array([0, 31, 32, 63, 1023, 1024, edge - 1, edge, n - 1]),
        12: np.arange(4096, 4096 + 32),                                  # exactly one word
        13: np.array([5, 5 + 64, 5 + 2 * 64, 700_000, 700_001, n - 2]),
        14: np.arange(edge + 1000, edge + 1000 + 300, 3),
    }
    for value, rows in groups.items():
        sig[:, rows, 0] = value
    sig[1, groups[12], 0] = 15                                            # table 1 splits one group in two
    sig[1, groups[12][::2], 0] = 16
    qsig = np.zeros((T, nq, H), dtype=np.uint8)
    for i, value in enumerate([10, 11, 12, 13, 14, 15, 16, 0, 1, 200, 12, 10]):
        qsig[:, i, 0] = value
    qsig[2, 10, 0] = 13                                                   # different small buckets per table
    qsig[0, 11, 0] = 1                                                    # a dense span beside sparse ones
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_index(qsig, ih), c_oracle.query_index_c(qsig, c_oracle.fit_index_c(sig, H)))
    ctx.free_index(ih)


@pytest.mark.parametrize("compact", [1, 0])
@pytest.mark.parametrize("cap", [0, 64, 8])
@pytest.mark.parametrize("n", [3000, 70_000])
def test_core_query_two_level_bitmap(ctx, c_oracle, monkeypatch, n, cap, compact):
    """The de-duplication kernel for queries with few candidates for the row range, forced on a small
    index: one bit per block of 32 rows, the non-empty blocks ranked, one word of row bits per ranked
    block.  Rows at both ends of a block, of a level-1 word (1024 rows) and of the index; a bucket of
    consecutive rows (blocks filled completely: a read-out step with more rows than its place holds is
    stored from registers); queries without candidates; tables that repeat each other's rows.  With a
    level 2 of 64 or 8 entries the queries take many rank ranges (counted first, then stored).  `compact`:
    the kernel is handed the list of queries that matched a bucket (the way it runs inside one bitmap
    pass) or every query."""
    _announce("two_level_bitmap", n, cap, compact)
    monkeypatch.setenv("CULSH_DEDUP_SPARSE", "1")
    monkeypatch.setenv("CULSH_DEDUP_COMPACT", str(compact))
    if cap:
        monkeypatch.setenv("CULSH_DEDUP_SPARSE_CAP", str(cap))
    rng = np.random.default_rng(1000 + n + cap)
    T, nq, H = 7, 300, 2
    sig = rng.integers(0, 12, size=(T, n, H)).astype(np.uint8)             # ~n/144 rows per bucket
    edges = np.array([0, 31, 32, 63, 1023, 1024, 1055, n - 33, n - 32, n - 1])
    sig[:, edges, 0] = 50
    run = np.arange(n // 2, n // 2 + 1500)                                  # 1500 consecutive rows: full blocks
    sig[:3, run, :] = 60
    sig[3:, run[::2], :] = 60                                               # other tables hold half of them
    qsig = rng.integers(0, 12, size=(T, nq, H)).astype(np.uint8)
    qsig[:, ::7, :] = 200                                                   # no candidates
    qsig[:, 1::7, 0] = 50                                                   # the edge rows (only)
    qsig[:, 2::7, :] = 60                                                   # the dense run
    qsig[:2, 3::7, :] = 60                                                  # dense run in two tables, random buckets in the rest
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    exp = c_oracle.query_index_c(qsig, c_oracle.fit_index_c(sig, H))
    assert_candidates_match(ctx.core_query_index(qsig, ih), exp)
    assert_candidates_match(ctx.core_query_index(qsig, ih), exp)            # output sized from the first call
    ctx.free_index(ih)


@pytest.mark.parametrize("T,n,nq", [(100, 5000, 150), (1, 2_200_000, 40), (5, 2_200_000, 64)])
def test_core_query_two_level_bitmap_shapes(ctx, c_oracle, monkeypatch, T, n, nq):
    """The two-level kernel with more tables than a wavefront has lanes, with one table, and on a row
    range of more than 2^20 rows (several level-1 words per thread), where it is chosen without being
    forced; the last row of the index is a candidate."""
    _announce("two_level_bitmap_shapes", T, n)
    if n < (1 << 20):
        monkeypatch.setenv("CULSH_DEDUP_SPARSE", "1")
    rng = np.random.default_rng(T + n)
    H = 2
    sig = rng.integers(0, 60, size=(T, n, H)).astype(np.uint8)
    sig[:, n - 1, :] = 100
    sig[:, n // 3, :] = 100
    qsig = rng.integers(0, 60, size=(T, nq, H)).astype(np.uint8)
    qsig[:, 5, :] = 100
    qsig[:, 6, :] = 255
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    exp = c_oracle.query_index_c(qsig, c_oracle.fit_index_c(sig, H))
    for _ in range(2):                                                      # second call: output sized from the first
        assert_candidates_match(ctx.core_query_index(qsig, ih), exp)
    ctx.free_index(ih)


def _kernels_run(ctx, fn):
    """Names of the library's kernels that `fn` launches (per-kernel event timing switched on around it)."""
    import ctypes as C

    from culsh_amd import _lib as L

    L.check(ctx.lib.culsh_profile_enable(ctx.h, 1))
    L.check(ctx.lib.culsh_profile_reset(ctx.h))
    try:
        result = fn()
        names = set()
        for i in range(ctx.lib.culsh_profile_count(ctx.h)):
            name, ms, cnt = C.c_char_p(), C.c_double(), C.c_int64()
            L.check(ctx.lib.culsh_profile_get(ctx.h, i, C.byref(name), C.byref(ms), C.byref(cnt)))
            if cnt.value:
                names.add(name.value.decode())
    finally:
        L.check(ctx.lib.culsh_profile_enable(ctx.h, 0))
    return result, names


def test_core_query_with_next_to_no_candidates_takes_the_two_level_kernel(ctx, c_oracle):
    """Inside one bitmap pass the two-level kernel is chosen, unforced, when the queries bring fewer than
    one raw candidate per 2048 rows (sweeping the bitmap would be most of such a query's time); the same
    index queried with rows of a large bucket goes back to the bitmap kernel.  Both against the oracle."""
    _announce("few_candidates_two_level")
    rng = np.random.default_rng(77)
    T, n, nq, H = 4, 200_000, 500, 3
    sig = rng.integers(0, 40, size=(T, n, H)).astype(np.uint8)              # ~3 rows per bucket
    sig[:, : n // 4, :] = 90                                                # and one bucket of 50,000 rows
    qsig = rng.integers(0, 40, size=(T, nq, H)).astype(np.uint8)
    qsig[:, ::5, :] = 200                                                   # no candidates
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    cix = c_oracle.fit_index_c(sig, H)
    exp = c_oracle.query_index_c(qsig, cix)
    for _ in range(2):                                                      # second call: path chosen from the first call's figures
        got, names = _kernels_run(ctx, lambda: ctx.core_query_index(qsig, ih))
        assert_candidates_match(got, exp)
        assert "dedup_sparse_kernel" in names and not any(k.startswith("dedup_kernel") for k in names), names
    heavy = qsig.copy()
    heavy[:, ::2, :] = 90
    exp_heavy = c_oracle.query_index_c(heavy, cix)
    assert_candidates_match(ctx.core_query_index(heavy, ih), exp_heavy)     # outgrows what the earlier calls suggest: redone
    got, names = _kernels_run(ctx, lambda: ctx.core_query_index(heavy, ih))
    assert_candidates_match(got, exp_heavy)
    assert "dedup_sparse_kernel" not in names, names
    ctx.free_index(ih)


@pytest.mark.parametrize("seed", range(6))
def test_core_query_every_path_on_random_shapes(ctx, c_oracle, monkeypatch, seed):
    """One seeded random index and query set (tables, rows, bucket sizes, share of queries without a match
    and of repeated rows all drawn) through every de-duplication path the library has: the choice it makes
    by itself, the bitmap kernel with several passes, the two-level kernel with and without the list of
    matched queries and with a small level 2, and the count / scan / emit launches.  All against the oracle."""
    _announce("every_path", seed)
    rng = np.random.default_rng(4000 + seed)
    T = int(rng.choice([1, 3, 17, 64, 65, 130]))
    n = int(rng.choice([700, 5000, 40_000, 150_000]))
    H = 2
    values = int(rng.choice([3, 12, 40]))                                    # n / values^2 rows per bucket
    nq = int(rng.integers(1, 400))
    sig = rng.integers(0, values, size=(T, n, H)).astype(np.uint8)
    if T > 1:
        sig[T // 2] = sig[0]                                                 # two tables with the same buckets
    qsig = rng.integers(0, values, size=(T, nq, H)).astype(np.uint8)
    qsig[:, rng.random(nq) < rng.choice([0.0, 0.5, 0.95]), :] = 250          # queries that match nothing
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    exp = c_oracle.query_index_c(qsig, c_oracle.fit_index_c(sig, H))
    paths = [{}, {"CULSH_DEDUP_WPT": "1"}, {"CULSH_DEDUP_SPARSE": "1"}, {"CULSH_DEDUP_SPARSE": "1", "CULSH_DEDUP_COMPACT": "0"},
             {"CULSH_DEDUP_SPARSE": "1", "CULSH_DEDUP_SPARSE_CAP": "32"}, {"CULSH_DEDUP_TWO_PASS": "1"},
             {"CULSH_QUERY_RAW_GUESS": "0"}]
    for env in paths:
        with monkeypatch.context() as m:
            for k, v in env.items():
                m.setenv(k, v)
            for _ in range(2):                                               # the second call sizes its output from the first
                assert_candidates_match(ctx.core_query_index(qsig, ih), exp)
    ctx.free_index(ih)


def test_core_query_two_level_bitmap_look_back_gives_up(ctx, monkeypatch):
    """The two-level kernel with no polls allowed in its chained scan: the call is redone with the
    count / scan / emit launches."""
    _announce("two_level_give_up")
    monkeypatch.setenv("CULSH_DEDUP_SPARSE", "1")
    monkeypatch.setenv("CULSH_DEDUP_SPIN_LIMIT", "0")
    rng = np.random.default_rng(15)
    T, n, nq, H = 6, 5000, 3000, 2
    sig = random_sigs(rng, T, n, H, "rplsh")
    qsig = random_sigs(rng, T, nq, H, "rplsh")
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, o.fit_index(sig, H)))
    ctx.free_index(ih)


def test_core_query_two_launch_path(ctx, monkeypatch):
    """The count / scan / emit path (taken for row ranges beyond one bitmap pass) on a small case."""
    _announce("two_launch_path")
    monkeypatch.setenv("CULSH_DEDUP_TWO_PASS", "1")
    rng = np.random.default_rng(91)
    T, n, nq, H = 5, 4000, 150, 2
    sig = random_sigs(rng, T, n, H, "rplsh")
    qsig = random_sigs(rng, T, nq, H, "rplsh")
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, o.fit_index(sig, H)))
    ctx.free_index(ih)


def test_core_query_after_look_back_gives_up(ctx, monkeypatch):
    """No polls allowed in the chained scan over the query counts: some workgroup gives up, the
    kernel still runs to its end, and the call is redone with the count / scan / emit launches."""
    _announce("dedup_give_up")
    monkeypatch.setenv("CULSH_DEDUP_SPIN_LIMIT", "0")
    rng = np.random.default_rng(5)
    T, n, nq, H = 6, 5000, 3000, 2
    sig = random_sigs(rng, T, n, H, "rplsh")
    qsig = random_sigs(rng, T, nq, H, "rplsh")
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, o.fit_index(sig, H)))
    ctx.free_index(ih)


@pytest.mark.parametrize("T,n,nq,H", [(90, 3000, 400, 3), (1024, 300, 40, 2)])
def test_core_query_more_than_64_tables(ctx, T, n, nq, H):
    """More tables than a wavefront has lanes (the spans of the next query are then not prefetched),
    up to the most an index may have (one thread per table)."""
    _announce("many_tables", T)
    rng = np.random.default_rng(6)
    sig = random_sigs(rng, T, n, H, "rplsh")
    qsig = random_sigs(rng, T, nq, H, "rplsh")
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, o.fit_index(sig, H)))
    ctx.free_index(ih)


def test_core_query_tables_that_overlap_completely(ctx, c_oracle):
    """Identical tables: the raw candidates outnumber the distinct ones eightfold, so the result
    array is cut down from its upper bound to the exact size."""
    _announce("overlapping_tables")
    rng = np.random.default_rng(17)
    T, n, nq, H = 8, 20000, 64, 1
    one = rng.integers(0, 2, size=(1, n, H), dtype=np.uint8)
    sig = np.ascontiguousarray(np.repeat(one, T, axis=0))
    qsig = np.ascontiguousarray(np.repeat(rng.integers(0, 2, size=(1, nq, H), dtype=np.uint8), T, axis=0))
    ih, _ = ctx.core_fit_index(sig, H)
    from abi import assert_candidates_match

    cix = c_oracle.fit_index_c(sig, H)
    got = ctx.core_query_index(qsig, ih)
    assert_candidates_match(got, c_oracle.query_index_c(qsig, cix))
    ctx.free_index(ih)


@pytest.mark.parametrize("kind", ["rplsh", "pslsh", "minhash"])
def test_core_fit_query(ctx, kind):
    """fit_query == fit + query on the same signatures (python/tests/test_rplsh.py:145-174)."""
    rng = np.random.default_rng(5)
    T, n, H = 4, 3000, 3
    sig = random_sigs(rng, T, n, H, kind)
    from abi import assert_candidates_match

    got = ctx.core_fit_query(sig, H)
    assert_candidates_match(got, o.fit_query(sig, H))
    ih, _ = ctx.core_fit_index(sig, H)
    again = ctx.core_query_index(sig, ih)
    for k in ("indices", "offsets", "counts"):
        np.testing.assert_array_equal(got[k], again[k])
    ctx.free_index(ih)


def test_candidates_merge_and_handles(ctx):
    """Candidates::merge (core/candidates.cuh:139-197) at the C ABI: parts of one query set, merged one
    after the other, equal the unbatched result; an empty accumulator takes the other object as it is
    (:144-148), an empty other changes nothing (:140-142), a part without any candidate still adds its
    queries.  Also the device-pointer, stream and synchronize exports."""
    from abi import assert_candidates_match
    from culsh_amd import _lib as L

    rng = np.random.default_rng(41)
    T, n, H, nq = 4, 3000, 3, 90
    sig = random_sigs(rng, T, n, H, "rplsh")
    qsig = random_sigs(rng, T, nq, H, "rplsh")
    ih, _ = ctx.core_fit_index(sig, H)
    exp_ix = o.fit_index(sig, H)
    whole = o.query_index(qsig, exp_ix)

    # three parts, chained: NULL accumulator first, then two appends
    cuts = [0, 25, 60, nq]
    acc = None
    for a, b in zip(cuts[:-1], cuts[1:]):
        part = ctx.core_query_index(np.ascontiguousarray(qsig[:, a:b]), ih, as_handle=True)
        acc = ctx.candidates_merge(acc, part)
    meta = ctx.candidates_meta(acc)
    assert meta["n_queries"] == nq and meta["n_total_candidates"] == whole.n_total_candidates
    # device pointers of the merged object hold the same arrays the copy calls return
    import torch

    def view(address, count, typestr):
        class Raw:
            __cuda_array_interface__ = {"shape": (count,), "typestr": typestr, "data": (address, False), "version": 2}
        return torch.as_tensor(Raw(), device="cuda").cpu().numpy()

    pi = ctx.candidates_device_ptr(acc, L.ARR_QUERY_INDICES)
    pc = ctx.candidates_device_ptr(acc, L.ARR_QUERY_COUNTS)
    po = ctx.candidates_device_ptr(acc, L.ARR_QUERY_OFFSETS)
    assert pi != 0 and pc != 0 and po != 0
    assert ctx.stream() != 0
    ctx.synchronize()
    np.testing.assert_array_equal(view(pi, whole.n_total_candidates, "<i4"), whole.query_candidate_indices)
    np.testing.assert_array_equal(view(pc, nq, "<i8").view(np.uint64), whole.query_candidate_counts)
    np.testing.assert_array_equal(view(po, nq + 1, "<i8").view(np.uint64), whole.query_candidate_offsets)
    assert_candidates_match(ctx.candidates_arrays(acc), whole)

    # empty accumulator object (no arrays) takes `other`; empty other leaves the accumulator as it is
    queries_without_bucket = np.full((T, 5, H), 7, dtype=np.uint8)   # byte 7 never occurs in 0/1 signatures
    none = ctx.core_query_index(queries_without_bucket, ih, as_handle=True)
    m = ctx.candidates_meta(none)
    assert m["n_queries"] == 5 and m["n_total_candidates"] == 0 and not m["is_empty"]
    assert ctx.candidates_device_ptr(none, L.ARR_QUERY_INDICES) == 0
    part = ctx.core_query_index(np.ascontiguousarray(qsig[:, :25]), ih, as_handle=True)
    acc = ctx.candidates_merge(none, part)       # a part with no candidate in front: offsets start with zeros
    got = ctx.candidates_arrays(acc)
    first = o.query_index(np.ascontiguousarray(qsig[:, :25]), exp_ix)
    assert got["n_queries"] == 30 and got["n_total_candidates"] == first.n_total_candidates
    np.testing.assert_array_equal(got["counts"], np.concatenate([np.zeros(5, np.uint64), first.query_candidate_counts]))
    np.testing.assert_array_equal(got["offsets"], np.concatenate([np.zeros(5, np.uint64), first.query_candidate_offsets]))
    np.testing.assert_array_equal(got["indices"], first.query_candidate_indices)
    # ... and behind: the oracle's merge says what comes out
    a = ctx.core_query_index(np.ascontiguousarray(qsig[:, :25]), ih, as_handle=True)
    b = ctx.core_query_index(queries_without_bucket, ih, as_handle=True)
    acc = ctx.candidates_merge(a, b)
    exp = o.merge(first, o.query_index(queries_without_bucket, exp_ix))
    assert_candidates_match(ctx.candidates_arrays(acc), exp)
    # NULL other: nothing happens, the accumulator handle stays valid
    a = ctx.core_query_index(np.ascontiguousarray(qsig[:, :25]), ih, as_handle=True)
    same = ctx.candidates_merge(a, None)
    assert same.value == a.value
    assert_candidates_match(ctx.candidates_arrays(same), first)
    ctx.free_index(ih)


# ---------------------------------------------------------------- whole path per family
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,T,H,nq", [(10000, 128, 16, 8, 100), (3000, 100, 8, 16, 64), (2000, 64, 3, 40, 50)])
def test_rplsh_fit_query_path(ctx, dtype, n, d, T, H, nq):
    """Config-1 shape (10000x128, 100 queries, 16 tables x 8 hashes, P from seed 42) and
    variants.  The bucket table must equal the oracle's table built from the GPU's own
    signatures (bit-exact given identical signatures); the GPU signatures must equal the
    float64 oracle's outside the band; candidate sets must have Jaccard >= 0.999."""
    _announce("rplsh_path", dtype.__name__, n, d, T, H, nq)
    rng = np.random.default_rng(1234)
    X = rng.standard_normal((n, d)).astype(dtype)
    Q = np.random.default_rng(4321).standard_normal((nq, d)).astype(dtype)
    P = np.random.default_rng(42).standard_normal((T * H, d)).astype(dtype)
    from abi import assert_candidates_match, assert_index_matches

    sig = ctx.rplsh_hash(X, P, T, H)
    qsig = ctx.rplsh_hash(Q, P, T, H)
    tol = TOL if dtype == np.float32 else 1e-12
    safe = o.rplsh_margin(X, P, T, H) > tol
    np.testing.assert_array_equal(sig[safe], o.rplsh_hash(X, P, T, H)[safe])

    ih = ctx.rplsh_fit(X, T, H, seed=42, P=P)
    exp_ix = o.fit_index(sig, H)
    got_ix = ctx.index_arrays(ih)
    assert_index_matches(got_ix, exp_ix)
    assert got_ix["n_features"] == d and got_ix["is_double"] == (dtype == np.float64)
    assert got_ix["sig_nbytes"] == H and got_ix["seed"] == 42
    np.testing.assert_array_equal(ctx.index_param(ih, 4, dtype), P.reshape(-1))

    got = ctx.rplsh_query(Q, ih)
    assert_candidates_match(got, o.query_index(qsig, exp_ix))
    # against the all-float64 oracle: per-query Jaccard
    ref = o.query_index(o.rplsh_hash(Q, P, T, H), o.fit_index(o.rplsh_hash(X, P, T, H), H))
    jac = []
    for q in range(nq):
        a = got["indices"][int(got["offsets"][q]):int(got["offsets"][q + 1])]
        b = ref.query_candidate_indices[int(ref.query_candidate_offsets[q]):int(ref.query_candidate_offsets[q + 1])]
        u = len(np.union1d(a, b))
        jac.append(1.0 if u == 0 else len(np.intersect1d(a, b)) / u)
    assert np.mean(jac) >= 0.999

    # batched == unbatched (python/tests/test_rplsh.py:177-209)
    for bs in (10, 50, nq, 7):
        bat = ctx.rplsh_query(Q, ih, batch_size=bs)
        for k in ("indices", "offsets", "counts"):
            np.testing.assert_array_equal(bat[k], got[k])

    # fit_query == fit + query(X) (python/tests/test_rplsh.py:145-174)
    m = min(n, 1500)
    fq = ctx.rplsh_fit_query(X[:m], T, H, seed=42, P=P)
    ih2 = ctx.rplsh_fit(X[:m], T, H, seed=42, P=P)
    qq = ctx.rplsh_query(X[:m], ih2)
    for k in ("indices", "offsets", "counts"):
        np.testing.assert_array_equal(fq[k], qq[k])
    ctx.free_index(ih)
    ctx.free_index(ih2)


@pytest.mark.parametrize("order", ["few_first", "many_first", "none_first"])
def test_batched_query_lists_written_in_place(ctx, order):
    """A batched query puts the batches' lists into one array that is sized after the first batch: later
    batches write behind what is there.  Batches that find far more per query than the first one do not
    fit and get arrays of their own (everything is put together at the end); a first batch that finds far
    more leaves the array oversized; a first batch without any candidate leaves none.  All equal the
    unbatched result, for several batch sizes (also one that does not divide the number of queries)."""
    _announce("batched_in_place", order)
    from abi import assert_candidates_match  # noqa: F401

    rng = np.random.default_rng(321)
    n, d, T, H = 6000, 24, 6, 10
    X = rng.standard_normal((n, d)).astype(np.float32)
    X[:2500] = X[0] + 1e-4 * rng.standard_normal((2500, d)).astype(np.float32)   # one crowd: 2500 rows per bucket
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    lone = rng.standard_normal((60, d)).astype(np.float32)                        # few candidates each
    crowd = np.repeat(X[:1], 90, axis=0) + 1e-4 * rng.standard_normal((90, d)).astype(np.float32)
    far = np.full((40, d), 0.0, np.float32)
    far[:, 0] = -1e6 * np.sign(P[:, 0].sum() + 1e-9)                              # (whatever it hashes to: a third kind)
    Q = {"few_first": np.concatenate([lone, crowd, lone[:7]]),
         "many_first": np.concatenate([crowd, lone, crowd[:5]]),
         "none_first": np.concatenate([far, lone, crowd])}[order]
    ih = ctx.rplsh_fit(X, T, H, seed=1, P=P)
    want = ctx.rplsh_query(Q, ih)
    assert want["n_total_candidates"] > 2500 * 50
    for bs in (50, 37, 20):
        got = ctx.rplsh_query(Q, ih, batch_size=bs)
        for k in ("counts", "offsets", "indices"):
            np.testing.assert_array_equal(got[k], want[k])
    ctx.free_index(ih)


@pytest.mark.parametrize("forced", ["", "sparse"])
def test_batched_query_with_next_to_no_candidates(ctx, monkeypatch, forced):
    """Batches whose queries mostly match nothing: inside a batch the two-level kernel works on the list of
    matched queries and takes its offsets from a scan, while the batches' lists still go into one array one
    behind the other.  Batched equals unbatched for several batch sizes; `sparse` forces that kernel for every
    batch, also the ones the library would give to the bitmap kernel."""
    _announce("batched_few_candidates", forced)
    if forced:
        monkeypatch.setenv("CULSH_DEDUP_SPARSE", "1")
    rng = np.random.default_rng(99)
    n, d, T, H = 150_000, 16, 5, 40                        # 40 hash bits per table: nearly every row alone in its bucket
    X = rng.standard_normal((n, d)).astype(np.float32)
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    Q = rng.standard_normal((900, d)).astype(np.float32)   # matches nothing, mostly
    Q[::9] = X[rng.integers(0, n, 100)]                    # every ninth query is a fitted row: at least itself
    ih = ctx.rplsh_fit(X, T, H, seed=1, P=P)
    want = ctx.rplsh_query(Q, ih)
    assert 100 <= want["n_total_candidates"] < 5000 and (want["counts"] == 0).sum() > 500
    for bs in (300, 128, 77):
        got = ctx.rplsh_query(Q, ih, batch_size=bs)
        for k in ("counts", "offsets", "indices"):
            np.testing.assert_array_equal(got[k], want[k])
    ctx.free_index(ih)


def test_rplsh_seeded_projection_matches_generator(ctx):
    """fit without an injected P draws it from the seed with the documented generator."""
    rng = np.random.default_rng(2)
    X = rng.standard_normal((500, 32)).astype(np.float32)
    ih = ctx.rplsh_fit(X, 4, 8, seed=7)
    P = ctx.index_param(ih, 4, np.float32).reshape(32, 32)
    np.testing.assert_allclose(P, o.generate_random_projections(7, 32, 32), rtol=2e-7, atol=0)
    from abi import assert_index_matches

    assert_index_matches(ctx.index_arrays(ih), o.fit_index(ctx.rplsh_hash(X, P, 4, 8), 8))
    ctx.free_index(ih)


def test_dtype_mismatch_is_an_error(ctx):
    """bindings.cu:58-60, 75-77"""
    X = np.random.default_rng(0).standard_normal((200, 16))
    ih32 = ctx.rplsh_fit(X.astype(np.float32), 2, 4)
    ih64 = ctx.rplsh_fit(X, 2, 4)
    with pytest.raises(RuntimeError, match="fitted with float32, but query is float64"):
        ctx.rplsh_query(X, ih32)
    with pytest.raises(RuntimeError, match="fitted with float64, but query is float32"):
        ctx.rplsh_query(X.astype(np.float32), ih64)
    ctx.free_index(ih32)
    ctx.free_index(ih64)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pslsh_fit_query_path(ctx, dtype):
    _announce("pslsh_path", dtype.__name__)
    n, d, T, H, nq, w = 5000, 128, 16, 8, 100, 4
    X = np.random.default_rng(1234).standard_normal((n, d)).astype(dtype)
    Q = (X[:nq] + 0.05 * np.random.default_rng(4321).standard_normal((nq, d))).astype(dtype)
    P, b = o.generate_random_projections_biases(42, T * H, d, w, dtype)
    from abi import assert_candidates_match, assert_index_matches

    sig = ctx.pslsh_hash(X, P, b, T, H)
    qsig = ctx.pslsh_hash(Q, P, b, T, H)
    ih = ctx.pslsh_fit(X, T, H, w, seed=42, P=P, b=b)
    exp_ix = o.fit_index(sig, H)
    got_ix = ctx.index_arrays(ih)
    assert_index_matches(got_ix, exp_ix)
    assert got_ix["sig_nbytes"] == 4 * H and got_ix["window_size"] == w
    got = ctx.pslsh_query(Q, ih)
    assert_candidates_match(got, o.query_index(qsig, exp_ix))
    assert got["n_total_candidates"] > 0
    for bs in (10, 50):
        bat = ctx.pslsh_query(Q, ih, batch_size=bs)
        for k in ("indices", "offsets", "counts"):
            np.testing.assert_array_equal(bat[k], got[k])
    fq = ctx.pslsh_fit_query(X[:1000], T, H, w, seed=42, P=P, b=b)
    ih2 = ctx.pslsh_fit(X[:1000], T, H, w, seed=42, P=P, b=b)
    qq = ctx.pslsh_query(X[:1000], ih2)
    for k in ("indices", "offsets", "counts"):
        np.testing.assert_array_equal(fq[k], qq[k])
    # seeded parameters follow the documented generator
    ih3 = ctx.pslsh_fit(X[:100], T, H, w, seed=42)
    np.testing.assert_allclose(ctx.index_param(ih3, 4, dtype), P.reshape(-1), rtol=3e-7)
    np.testing.assert_allclose(ctx.index_param(ih3, 5, dtype), b, rtol=3e-7)
    for h in (ih, ih2, ih3):
        ctx.free_index(h)


def test_pslsh_many_hashes_narrow_ranges(ctx):
    """896 hashes of two or three values each: rank keys of 56 words, the widest the signature restore
    kernel takes, with value tables that no longer fit into LDS beside them."""
    _announce("pslsh_many_hashes")
    n, d, T, H, nq, w = 400, 16, 2, 896, 40, 64
    rng = np.random.default_rng(8)
    X = rng.standard_normal((n, d)).astype(np.float32)
    Q = X[:nq].copy()
    P, b = o.generate_random_projections_biases(7, T * H, d, w, np.float32)
    from abi import assert_candidates_match, assert_index_matches

    sig = ctx.pslsh_hash(X, P, b, T, H)
    assert 2 <= int(sig.max()) - int(sig.min()) + 1 <= 3
    ih = ctx.pslsh_fit(X, T, H, w, seed=7, P=P, b=b)
    exp_ix = o.fit_index(sig, H)
    assert_index_matches(ctx.index_arrays(ih), exp_ix)
    assert_candidates_match(ctx.pslsh_query(Q, ih), o.query_index(ctx.pslsh_hash(Q, P, b, T, H), exp_ix))
    ctx.free_index(ih)


def test_minhash_fit_query_path(ctx):
    _announce("minhash_path")
    rng = np.random.default_rng(77)
    n, d, T, H, nq = 4000, 2000, 32, 4, 100
    indices, indptr = make_csr(rng, n, d, 30, empty_rows=(3, 9))
    # queries: perturbed copies of rows so that buckets are hit
    qrows = []
    for i in range(nq):
        r = indices[indptr[i]:indptr[i + 1]]
        keep = r[rng.random(len(r)) > 0.1]
        qrows.append(np.unique(np.concatenate([keep, rng.choice(d, 2)])))
    qindptr = np.concatenate([[0], np.cumsum([len(r) for r in qrows])]).astype(np.int32)
    qindices = np.concatenate(qrows).astype(np.int32)
    A, B = o.generate_hash_integers(42, T * H)
    from abi import assert_candidates_match, assert_index_matches

    sig = o.minhash_hash(indices, indptr, A, B, T, H)       # exact integers: oracle signatures
    qsig = o.minhash_hash(qindices, qindptr, A, B, T, H)
    ih = ctx.minhash_fit(indices, indptr, d, T, H, seed=42, A=A, B=B)
    exp_ix = o.fit_index(sig, H)
    got_ix = ctx.index_arrays(ih)
    assert_index_matches(got_ix, exp_ix)
    assert got_ix["sig_nbytes"] == 4 * H
    got = ctx.minhash_query(qindices, qindptr, ih)
    assert_candidates_match(got, o.query_index(qsig, exp_ix))
    assert got["n_total_candidates"] > nq // 2
    fq = ctx.minhash_fit_query(indices, indptr, d, T, H, seed=42, A=A, B=B)
    assert_candidates_match(fq, o.fit_query(sig, H))
    # seeded coefficients follow the documented generator, bit for bit
    ih2 = ctx.minhash_fit(indices, indptr, d, T, H, seed=42)
    np.testing.assert_array_equal(ctx.index_param(ih2, 6, np.uint32), A)
    np.testing.assert_array_equal(ctx.index_param(ih2, 7, np.uint32), B)
    ctx.free_index(ih)
    ctx.free_index(ih2)


@pytest.mark.parametrize("n,d,T,H,nnz", [(500, 5000, 32, 4, 50), (77, 300, 5, 3, 8), (64, 100000, 2, 130, 20)])
def test_minhash_compute_exact_mod_mersenne_prime(n, d, T, H, nnz):
    """The prime is a parameter of the hashing kernels: 2^31 - 1 instead of the reference's 2^32 - 5,
    against the oracle with the same prime; parameters at the ends of their ranges and parameters that are
    not normalised at all (any 32-bit value may be injected)."""
    _announce("minhash_mersenne", n, d, T, H, nnz)
    from abi import Ctx

    p31 = o.MINHASH_PRIME_MERSENNE
    rng = np.random.default_rng(n + H)
    indices, indptr = make_csr(rng, n, d, nnz, empty_rows=(0,))
    A, B = o.generate_hash_integers(9, T * H, p31)
    A[0], B[0] = p31 - 1, p31 - 1
    if T * H > 2:
        A[1], B[1] = 0xFFFFFFFF, 0xFFFFFFFE
    own = Ctx(0)
    try:
        with pytest.raises(RuntimeError):
            own.set_minhash_prime(4294967295)                     # neither of the two primes
        own.set_minhash_prime(p31)
        np.testing.assert_array_equal(own.minhash_compute(indices, indptr, A, B, T, H),
                                      o.minhash_hash(indices, indptr, A, B, T, H, p31))
        own.set_minhash_prime(o.MINHASH_PRIME)
        np.testing.assert_array_equal(own.minhash_compute(indices, indptr, A, B, T, H),
                                      o.minhash_hash(indices, indptr, A, B, T, H))
    finally:
        own.close()


@pytest.mark.parametrize("beyond", [False, True])
def test_minhash_fit_query_path_mod_mersenne_prime(c_oracle, beyond):
    """Fit, query and fit_query with the family taken modulo 2^31 - 1: bucket tables and candidate lists
    against the oracle on signatures of the same prime.  With rank keys (every column id below
    n_features; the column of a minimum is recovered through the multiplier's inverse modulo that prime)
    and with plain keys (`beyond`: some ids at or above n_features, found during the fit)."""
    _announce("minhash_path_mersenne", beyond)
    from abi import Ctx, assert_candidates_match, assert_index_matches

    p31 = o.MINHASH_PRIME_MERSENNE
    rng = np.random.default_rng(78)
    n, d, T, H, nq = 6000, 3000, 16, 4, 200
    indices, indptr = make_csr(rng, n, d, 25, empty_rows=(3, 9))
    if beyond:
        indices = indices.copy()
        indices[rng.integers(0, len(indices), 40)] = d + 5
    qrows = []
    for i in range(nq):
        r = indices[indptr[i]:indptr[i + 1]]
        keep = r[rng.random(len(r)) > 0.1]
        qrows.append(np.unique(np.concatenate([keep, rng.choice(d, 2)])))
    qindptr = np.concatenate([[0], np.cumsum([len(r) for r in qrows])]).astype(np.int32)
    qindices = np.concatenate(qrows).astype(np.int32)
    own = Ctx(0)
    try:
        own.set_minhash_prime(p31)
        ih = own.minhash_fit(indices, indptr, d, T, H, seed=42)   # seeded parameters, normalised for this prime
        A, B = o.generate_hash_integers(42, T * H, p31)
        np.testing.assert_array_equal(own.index_param(ih, 6, np.uint32), A)
        np.testing.assert_array_equal(own.index_param(ih, 7, np.uint32), B)
        assert own.index_minhash_prime(ih) == p31
        sig = c_oracle.minhash_hash(indices, indptr, A, B, T, H, p31)
        qsig = c_oracle.minhash_hash(qindices, qindptr, A, B, T, H, p31)
        assert not np.array_equal(sig, c_oracle.minhash_hash(indices, indptr, A, B, T, H))   # the prime matters
        cix = c_oracle.fit_index_c(sig, H)
        assert_index_matches(own.index_arrays(ih), cix.to_numpy(n))
        own.set_minhash_prime(o.MINHASH_PRIME)                    # a query hashes with its index's prime
        got = own.minhash_query(qindices, qindptr, ih)
        assert_candidates_match(got, c_oracle.query_index_c(qsig, cix))
        assert got["n_total_candidates"] > nq // 2
        own.set_minhash_prime(p31)
        assert_candidates_match(own.minhash_fit_query(indices, indptr, d, T, H, seed=42, A=A, B=B),
                                c_oracle.fit_query(sig, H))
        own.free_index(ih)
    finally:
        own.close()


def test_pslsh_query_values_never_seen_at_fit(ctx):
    """p-stable keys are stored as per-hash ranks of the values seen at fit time; a query
    hash outside that range (or inside it but never seen) must simply match no bucket."""
    n, d, T, H, w = 3000, 32, 8, 4, 4
    X = np.random.default_rng(5).standard_normal((n, d)).astype(np.float32)
    P, b = o.generate_random_projections_biases(3, T * H, d, w, np.float32)
    Q = np.concatenate([X[:50], 40.0 * X[50:100], -40.0 * X[100:150]]).astype(np.float32)
    from abi import assert_candidates_match, assert_index_matches

    sig, qsig = ctx.pslsh_hash(X, P, b, T, H), ctx.pslsh_hash(Q, P, b, T, H)
    assert qsig.max() > sig.max() and qsig.min() < sig.min()
    ih = ctx.pslsh_fit(X, T, H, w, P=P, b=b)
    exp_ix = o.fit_index(sig, H)
    assert_index_matches(ctx.index_arrays(ih), exp_ix)
    got = ctx.pslsh_query(Q, ih)
    assert_candidates_match(got, o.query_index(qsig, exp_ix))
    assert got["counts"][:50].min() >= 1 and got["counts"][50:].sum() < got["counts"][:50].sum()
    # the same index queried through the signature-level entry point
    assert_candidates_match(ctx.core_query_index(qsig, ih), o.query_index(qsig, exp_ix))
    ctx.free_index(ih)


def test_pslsh_wide_value_range_keeps_plain_keys(ctx):
    """Hash values spread over more than 4095 distinct values per hash function: keys stay
    the byte-order words of the int32 hashes (32 * H bits)."""
    n, d, T, H = 4000, 16, 3, 2
    rng = np.random.default_rng(6)
    X = rng.standard_normal((n, d)).astype(np.float32)
    P = (rng.standard_normal((T * H, d)) * 3000.0).astype(np.float32)
    b = rng.uniform(0.1, 1.0, size=T * H).astype(np.float32)
    from abi import assert_candidates_match, assert_index_matches

    sig = ctx.pslsh_hash(X, P, b, T, H)
    assert sig.max() - sig.min() > 8192
    sig[:, 1::2] = sig[:, 0::2]      # make buckets of two rows: signatures of odd rows copy even rows
    X[1::2] = X[0::2]
    ih = ctx.pslsh_fit(X, T, H, 1, P=P, b=b)
    exp_ix = o.fit_index(sig, H)
    assert_index_matches(ctx.index_arrays(ih), exp_ix)
    assert_candidates_match(ctx.pslsh_query(X[:200], ih), o.query_index(sig[:, :200], exp_ix))
    ctx.free_index(ih)


def test_object_memory_is_reused_and_trimmed(ctx):
    """Index and candidate arrays come from a cache of freed blocks: results must not depend on
    whether a block is fresh or reused, and trimming the cache must leave everything working."""
    _announce("memory_pool")
    rng = np.random.default_rng(3)
    T, n, nq, H = 4, 3000, 100, 3
    sig = random_sigs(rng, T, n, H, "rplsh")
    qsig = random_sigs(rng, T, nq, H, "rplsh")
    exp_ix = o.fit_index(sig, H)
    exp = o.query_index(qsig, exp_ix)
    from abi import assert_candidates_match, assert_index_matches

    for round_ in range(3):
        ih, _ = ctx.core_fit_index(sig, H)
        assert_index_matches(ctx.index_arrays(ih), exp_ix)
        assert_candidates_match(ctx.core_query_index(qsig, ih), exp)
        ctx.free_index(ih)
        if round_ == 1:
            ctx.lib.culsh_memory_trim()


def test_full_size_invariants(ctx):
    """Benchmark configuration 2 of the reference at its real size (1M x 128, 32 tables x 16 hashes, 10k queries): properties
    that hold for any correct index / candidate set, checked on everything, plus a brute-force
    comparison for a sample of queries."""
    _announce("full_size")
    n, d, nq, T, H = 1_000_000, 128, 10_000, 32, 16
    rng = np.random.default_rng(2024)
    X = np.clip(np.floor(rng.gamma(0.5, 30.0, size=(n, d))), 0, 255).astype(np.float32)
    rows = rng.integers(0, n, size=nq)
    Q = np.clip(X[rows] + rng.normal(0.0, 3.0, size=(nq, d)), 0, 255).astype(np.float32)
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    ih = ctx.rplsh_fit(X, T, H, P=P)
    ix = ctx.index_arrays(ih)
    N = n * T
    tbo, bco = ix["table_bucket_offsets"].astype(np.int64), ix["bucket_candidate_offsets"].astype(np.int64)
    B = int(ix["n_total_buckets"])
    cand = ix["all_candidate_indices"]
    assert tbo[0] == 0 and tbo[-1] == B and np.all(np.diff(tbo) > 0)
    assert bco[0] == 0 and bco[-1] == N and np.all(np.diff(bco) > 0)
    assert np.all(bco[tbo[:-1]] == np.arange(T) * n)            # a table's first bucket starts its segment
    # every table holds every row exactly once
    for t in range(T):
        assert np.array_equal(np.bincount(cand[t * n:(t + 1) * n], minlength=n), np.ones(n, dtype=np.int64))
    # rows ascend inside a bucket: the only descents of the candidate array are at bucket starts
    descents = np.flatnonzero(np.diff(cand.astype(np.int64)) < 0) + 1
    assert np.all(np.isin(descents, bco))
    # bucket signatures strictly ascend (byte order) inside a table
    sig = ix["all_bucket_signatures"].reshape(B, H)
    keys = sig.astype(np.int64) @ (1 << np.arange(H - 1, -1, -1)).astype(np.int64)   # H = 16 sign bytes as a number
    inc = np.diff(keys) > 0
    inc[tbo[1:-1] - 1] = True                                    # table boundaries may descend
    assert np.all(inc)
    # signatures agree with the GPU's own hash of the rows they contain (first row of a sample of buckets)
    gsig = ctx.rplsh_hash(X[:20000], P, T, H)                    # [T][20000][H]
    bucket_of_pos = np.searchsorted(bco, np.arange(0, N, 997), side="right") - 1
    for pos, b in zip(np.arange(0, N, 997)[:4000], bucket_of_pos[:4000]):
        r, t = int(cand[pos]), int(pos // n)
        if r < 20000:
            assert np.array_equal(sig[b], gsig[t, r])
    # queries
    got = ctx.rplsh_query(Q, ih)
    off, idx = got["offsets"].astype(np.int64), got["indices"]
    assert off[0] == 0 and off[-1] == len(idx) and np.all(np.diff(off) >= 0)
    assert np.array_equal(np.diff(off), got["counts"].astype(np.int64))
    inside = np.ones(len(idx), dtype=bool)
    inside[off[1:-1][off[1:-1] < len(idx)]] = False              # first element of the next query
    assert np.all((np.diff(idx.astype(np.int64)) > 0) | ~inside[1:])   # ascending and duplicate-free per query
    assert idx.min() >= 0 and idx.max() < n
    # brute force for a sample: union over tables of the rows in the bucket that matches the query's signature
    qsig = ctx.rplsh_hash(Q[:64], P, T, H)
    for q in range(0, 64, 7):
        exp = []
        for t in range(T):
            lo, hi = tbo[t], tbo[t + 1]
            hit = np.flatnonzero((sig[lo:hi] == qsig[t, q]).all(axis=1))
            if len(hit):
                b = lo + hit[0]
                exp.append(cand[bco[b]:bco[b + 1]])
        exp = np.unique(np.concatenate(exp)) if exp else np.zeros(0, np.int32)
        np.testing.assert_array_equal(idx[off[q]:off[q + 1]], exp)
    ctx.free_index(ih)


def _index_properties(ix, n, T, S):
    """Properties of any correct index (core/fit.cuh:222-374): offsets with their terminators, every table a
    permutation of the rows, rows ascending inside a bucket, bucket signatures strictly ascending in byte
    order inside a table."""
    N = n * T
    tbo, bco = ix["table_bucket_offsets"].astype(np.int64), ix["bucket_candidate_offsets"].astype(np.int64)
    B = int(ix["n_total_buckets"])
    cand = ix["all_candidate_indices"]
    assert ix["sig_nbytes"] == S and ix["n_total_candidates"] == N
    assert tbo[0] == 0 and tbo[-1] == B and np.all(np.diff(tbo) > 0)
    assert bco[0] == 0 and bco[-1] == N and np.all(np.diff(bco) > 0)
    assert np.all(bco[tbo[:-1]] == np.arange(T) * n)            # a table's first bucket starts its segment
    for t in range(T):
        assert np.array_equal(np.bincount(cand[t * n:(t + 1) * n], minlength=n), np.ones(n, dtype=np.int64))
    descents = np.flatnonzero(np.diff(cand.astype(np.int64)) < 0) + 1
    assert np.all(np.isin(descents, bco))
    # byte-lexicographic order = numeric order of the big-endian words of a signature
    assert S % 8 == 0
    words = ix["all_bucket_signatures"].reshape(B, S).view(">u8").astype(np.uint64)   # [B][S/8]
    differs = words[1:] != words[:-1]
    first = np.argmax(differs, axis=1)
    rows_idx = np.arange(B - 1)
    ascending = differs.any(axis=1) & (words[1:][rows_idx, first] > words[:-1][rows_idx, first])
    ascending[tbo[1:-1] - 1] = True                              # table boundaries may descend
    assert np.all(ascending)


def _candidate_properties(got, n):
    off, idx = got["offsets"].astype(np.int64), got["indices"]
    assert off[0] == 0 and off[-1] == len(idx) and np.all(np.diff(off) >= 0)
    assert np.array_equal(np.diff(off), got["counts"].astype(np.int64))
    if len(idx):
        inside = np.ones(len(idx), dtype=bool)
        inside[off[1:-1][off[1:-1] < len(idx)]] = False          # first element of the next query
        assert np.all((np.diff(idx.astype(np.int64)) > 0) | ~inside[1:])   # ascending and duplicate-free per query
        assert idx.min() >= 0 and idx.max() < n


def test_config3_full_size(ctx, c_oracle):
    """Benchmark configuration 3 at its real size: p-stable LSH, 1,000,000 x 128 N(0,1) rows, 16 tables x 8
    hashes, window 4 (P = a / 4, b in (0, 1]; pslsh/hash.cuh:25-47, 59-89) - some 16M buckets, rank-compressed
    keys.  Properties on everything; the whole index and the candidate lists bit-exact against the C oracle
    given the GPU's signatures; signatures against the float64 oracle outside the band on a sample of rows.
    Queries: the configuration's own N(0,1) queries (hardly any candidate) and fitted rows with a little
    noise (candidates for most)."""
    _announce("config3_full_size")
    from abi import assert_candidates_match, assert_index_matches

    n, d, nq, T, H, w = 1_000_000, 128, 10_000, 16, 8, 4
    rng = np.random.default_rng(303)
    X = rng.standard_normal((n, d), dtype=np.float32)
    Q = rng.standard_normal((nq, d), dtype=np.float32)
    near = X[rng.integers(0, n, size=nq)] + rng.normal(0.0, 0.02, size=(nq, d)).astype(np.float32)
    P = (rng.standard_normal((T * H, d)) / w).astype(np.float32)
    b = (1.0 - rng.random(T * H)).astype(np.float32)             # (0, 1]
    ih = ctx.pslsh_fit(X, T, H, w, P=P, b=b)
    ix = ctx.index_arrays(ih)
    _index_properties(ix, n, T, 4 * H)
    sig = ctx.pslsh_hash(X, P, b, T, H)                           # [T][n][H] int32
    rows = rng.integers(0, n, size=3000)
    safe = o.pslsh_margin(X[rows], P, b, T, H) > TOL
    assert safe.mean() > 0.999
    np.testing.assert_array_equal(sig[:, rows][safe], o.pslsh_hash(X[rows], P, b, T, H)[safe])
    cix = c_oracle.fit_index_c(sig, H)
    assert_index_matches(ix, cix.to_numpy(n))
    del sig
    for queries, expect_hits in ((Q, False), (near, True)):
        got = ctx.pslsh_query(queries, ih)
        _candidate_properties(got, n)
        qsig = ctx.pslsh_hash(queries, P, b, T, H)
        assert_candidates_match(got, c_oracle.query_index_c(qsig, cix))
        if expect_hits:
            assert (got["counts"] > 0).mean() > 0.5
    ctx.free_index(ih)


def test_config4_full_size(ctx, c_oracle):
    """Benchmark configuration 4 at its real size: MinHash, 1,000,000 rows over 50,000 columns, Poisson(50)
    distinct columns per row drawn from a Zipf(1.1) law, 32 tables x 4 hashes, prime 4294967291
    (minhash/hash.cuh:17, 69-128) - some 25M buckets, rank-coded 64-bit keys, 8 radix passes.  Signatures are
    exact integers: the GPU's equal the oracle's on a sample of rows; the whole index and the candidate lists
    are bit-exact against the C oracle given the signatures."""
    _announce("config4_full_size")
    import torch

    from abi import assert_candidates_match, assert_index_matches
    from culsh_amd.benchmark import _zipf_sets

    n, d, nq, T, H = 1_000_000, 50_000, 10_000, 32, 4
    g = torch.Generator(device="cuda")
    g.manual_seed(404)
    Xd, Qd = _zipf_sets(torch, n, d, nq, g)
    xi, xp = Xd.indices.cpu().numpy(), Xd.indptr.cpu().numpy()
    qi, qp = Qd.indices.cpu().numpy(), Qd.indptr.cpu().numpy()
    del Xd, Qd
    nnz = np.diff(xp)
    assert 49.5 < nnz.mean() < 50.5 and 6.5 < nnz.std() < 7.6 and nnz.min() >= 1 and xi.max() < d   # Poisson(50)
    starts = np.ones(len(xi), dtype=bool)
    starts[xp[1:-1]] = False
    assert np.all((np.diff(xi.astype(np.int64)) > 0) | ~starts[1:])   # distinct, ascending columns inside a row
    top = np.bincount(xi, minlength=d)
    assert top[0] > 0.99 * n and top[10] > 2 * top[100] > 4 * top[1000] > 0   # heavy head of the Zipf law: nearly every row holds column 0
    A, B = o.generate_hash_integers(42, T * H)
    ih = ctx.minhash_fit(xi, xp, d, T, H, seed=42, A=A, B=B)
    ix = ctx.index_arrays(ih)
    _index_properties(ix, n, T, 4 * H)
    sig = ctx.minhash_compute(xi, xp, A, B, T, H)                 # [T][n][H] uint32
    rows = np.random.default_rng(5).integers(0, n, size=2000)
    sub_ptr = np.concatenate([[0], np.cumsum(nnz[rows])]).astype(np.int32)
    sub_idx = np.concatenate([xi[xp[r]:xp[r + 1]] for r in rows]).astype(np.int32)
    np.testing.assert_array_equal(sig[:, rows], o.minhash_hash(sub_idx, sub_ptr, A, B, T, H))
    cix = c_oracle.fit_index_c(sig, H)
    assert_index_matches(ix, cix.to_numpy(n))
    del sig
    got = ctx.minhash_query(qi, qp, ih)
    _candidate_properties(got, n)
    qsig = ctx.minhash_compute(qi, qp, A, B, T, H)
    np.testing.assert_array_equal(qsig, c_oracle.minhash_hash(qi, qp, A, B, T, H))
    assert_candidates_match(got, c_oracle.query_index_c(qsig, cix))
    assert got["n_total_candidates"] > 0
    ctx.free_index(ih)


def test_item_count_just_below_2_31(ctx):
    """n_samples * n_hash_tables = 2,097,152,000 items, the most the 32-bit offsets of the index hold
    (limit 2^31): 2M rows x 8 features into 1000 tables x 4 hashes.  Everything is checked on the device
    (torch as plumbing): a permutation of the rows in the first, a middle and the last table, rows
    ascending inside buckets, offsets that end at the item count, and four queries against a brute-force
    union over all 1000 tables computed from the stage-level signatures."""
    import ctypes as C

    import torch

    from culsh_amd import _lib as L
    from culsh_amd.abi import dev, hp, ptr

    _announce("items_just_below_2_31")
    n, d, T, H, nq = 1 << 21, 8, 1000, 4, 4
    rng = np.random.default_rng(2031)
    X = rng.standard_normal((n, d)).astype(np.float32)
    P = rng.standard_normal((T * H, d)).astype(np.float32)
    qrows = np.array([0, 123_457, n // 2 + 1, n - 1])
    dX, dP = dev(X), dev(P)
    dQ = dev(np.ascontiguousarray(X[qrows]))
    lib = ctx.lib
    ih = C.c_void_p()
    L.check(lib.culsh_rplsh_fit_f32(ctx.h, ptr(dX), n, d, T, H, 1, hp(P), C.byref(ih)))
    try:
        m = L.IndexMeta()
        L.check(lib.culsh_index_get_meta(ih, C.byref(m)))
        N = n * T
        assert m.n_total_candidates == N and N < 2 ** 31 and 0 < m.n_total_buckets <= T * (1 << H)
        B = int(m.n_total_buckets)

        def on_device(which, count, dtype):
            out = torch.empty(count, dtype=dtype, device="cuda")
            L.check(lib.culsh_index_copy_array(ctx.h, ih, which, ptr(out), out.numel() * out.element_size(), 1))
            return out

        tbo = on_device(L.ARR_TABLE_BUCKET_OFFSETS, T + 1, torch.int32).cpu().numpy().astype(np.int64)
        assert tbo[0] == 0 and tbo[-1] == B and (np.diff(tbo) > 0).all()
        bco = on_device(L.ARR_BUCKET_CANDIDATE_OFFSETS, B + 1, torch.int32).to(torch.int64)
        assert int(bco[0]) == 0 and int(bco[-1]) == N and bool((bco[1:] > bco[:-1]).all())
        # every table's buckets cover exactly its n items
        ends = bco[torch.from_numpy(tbo).cuda()]
        assert bool((ends == torch.arange(T + 1, device="cuda", dtype=torch.int64) * n).all())
        cand = on_device(L.ARR_CANDIDATE_INDICES, N, torch.int32)
        for t in (0, T // 2, T - 1):
            rows = cand[t * n:(t + 1) * n].to(torch.int64)
            assert int(rows.min()) == 0 and int(rows.max()) == n - 1
            assert bool((torch.bincount(rows, minlength=n) == 1).all())              # a permutation of the rows
            starts = torch.zeros(n, dtype=torch.bool, device="cuda")
            b0, b1 = int(tbo[t]), int(tbo[t + 1])
            starts[(bco[b0:b1] - t * n)] = True
            assert bool(((rows[1:] > rows[:-1]) | starts[1:]).all())                 # ascending inside every bucket
            del rows, starts
        del cand
        # four queries (rows of X) against brute force over all tables
        sig = torch.empty(T * n * H, dtype=torch.uint8, device="cuda")
        L.check(lib.culsh_rplsh_hash_f32(ctx.h, ptr(dX), ptr(dP), n, d, T, H, ptr(sig)))
        sig = sig.view(T, n, H)
        ch = C.c_void_p()
        L.check(lib.culsh_rplsh_query_f32(ctx.h, ptr(dQ), nq, ih, -1, C.byref(ch)))
        got = ctx.candidates_arrays(ch)
        assert got["offsets"][0] == 0 and got["offsets"][-1] == got["n_total_candidates"]
        for i, r in enumerate(qrows):
            same = torch.zeros(n, dtype=torch.bool, device="cuda")
            for t0 in range(0, T, 100):
                part = sig[t0:t0 + 100]
                same |= (part == part[:, r:r + 1, :]).all(dim=2).any(dim=0)
            exp = torch.nonzero(same).flatten().cpu().numpy().astype(np.int32)
            lo, hi = int(got["offsets"][i]), int(got["offsets"][i + 1])
            assert got["counts"][i] == hi - lo == exp.size and r in exp
            np.testing.assert_array_equal(got["indices"][lo:hi], exp)
    finally:
        lib.culsh_index_free(ih)


@pytest.mark.parametrize("family", ["pslsh", "minhash"])
def test_item_count_just_below_2_31_wide_key_families(ctx, family):
    """The same size (2^21 rows x 1000 tables) for the families with rank-compressed keys, two hashes per
    table: index invariants on the device, and four queries against a brute-force union over all tables
    computed from the stage-level hashes."""
    import ctypes as C

    import torch

    from culsh_amd import _lib as L
    from culsh_amd.abi import dev, hp, ptr

    _announce("items_just_below_2_31", family)
    n, T, H, nq = 1 << 21, 1000, 2, 4
    rng = np.random.default_rng(2032)
    qrows = np.array([1, 654_321, n // 2, n - 1])
    lib = ctx.lib
    ih, ch = C.c_void_p(), C.c_void_p()
    if family == "pslsh":
        d, w = 8, 4
        X = rng.standard_normal((n, d)).astype(np.float32)
        P, b = o.generate_random_projections_biases(11, T * H, d, w, np.float32)
        dX, dP, db = dev(X), dev(P), dev(b)
        dQ = dev(np.ascontiguousarray(X[qrows]))
        sig = torch.empty(T * n * H, dtype=torch.int32, device="cuda")
        L.check(lib.culsh_pslsh_hash_f32(ctx.h, ptr(dX), ptr(dP), ptr(db), n, d, T, H, ptr(sig)))
        L.check(lib.culsh_pslsh_fit_f32(ctx.h, ptr(dX), n, d, T, H, w, 11, hp(P), hp(b), C.byref(ih)))
        L.check(lib.culsh_pslsh_query_f32(ctx.h, ptr(dQ), nq, ih, -1, C.byref(ch)))
    else:
        d = 1000
        # six distinct columns per row: base + k * stride (mod d) with 5 * stride < d, sorted per row
        base, stride = rng.integers(0, d, size=(n, 1)), rng.integers(1, d // 6, size=(n, 1))
        indices = np.sort((base + np.arange(6) * stride) % d, axis=1).astype(np.int32).reshape(-1)
        indptr = (np.arange(n + 1, dtype=np.int64) * 6).astype(np.int32)
        A, B = o.generate_hash_integers(12, T * H)
        dI, dPtr, dA, dB = dev(indices), dev(indptr), dev(A), dev(B)
        qi = np.concatenate([indices[indptr[r]:indptr[r + 1]] for r in qrows]).astype(np.int32)
        qp = np.concatenate([[0], np.cumsum([indptr[r + 1] - indptr[r] for r in qrows])]).astype(np.int32)
        dqi, dqp = dev(qi), dev(qp)
        sig = torch.empty(T * n * H, dtype=torch.int32, device="cuda")   # uint32 values, compared for equality only
        L.check(lib.culsh_minhash_compute(ctx.h, ptr(dI), ptr(dPtr), ptr(dA), ptr(dB), n, T, H, ptr(sig)))
        L.check(lib.culsh_minhash_fit(ctx.h, ptr(dI), ptr(dPtr), n, d, T, H, 12, hp(A), hp(B), C.byref(ih)))
        L.check(lib.culsh_minhash_query(ctx.h, ptr(dqi), ptr(dqp), nq, ih, C.byref(ch)))
    try:
        m = L.IndexMeta()
        L.check(lib.culsh_index_get_meta(ih, C.byref(m)))
        N, Bk = n * T, int(m.n_total_buckets)
        assert m.n_total_candidates == N and m.sig_nbytes == 4 * H

        def on_device(which, count, dtype):
            out = torch.empty(count, dtype=dtype, device="cuda")
            L.check(lib.culsh_index_copy_array(ctx.h, ih, which, ptr(out), out.numel() * out.element_size(), 1))
            return out

        tbo = on_device(L.ARR_TABLE_BUCKET_OFFSETS, T + 1, torch.int32).cpu().numpy().astype(np.int64)
        bco = on_device(L.ARR_BUCKET_CANDIDATE_OFFSETS, Bk + 1, torch.int32).to(torch.int64)
        assert tbo[0] == 0 and tbo[-1] == Bk and int(bco[0]) == 0 and int(bco[-1]) == N
        assert bool((bco[1:] > bco[:-1]).all())
        assert bool((bco[torch.from_numpy(tbo).cuda()] == torch.arange(T + 1, device="cuda", dtype=torch.int64) * n).all())
        cand = on_device(L.ARR_CANDIDATE_INDICES, N, torch.int32)
        for t in (0, T - 1):
            rows = cand[t * n:(t + 1) * n].to(torch.int64)
            assert bool((torch.bincount(rows, minlength=n) == 1).all())
            starts = torch.zeros(n, dtype=torch.bool, device="cuda")
            starts[(bco[int(tbo[t]):int(tbo[t + 1])] - t * n)] = True
            assert bool(((rows[1:] > rows[:-1]) | starts[1:]).all())
            del rows, starts
        del cand
        sig = sig.view(T, n, H)
        got = ctx.candidates_arrays(ch)
        ch = None
        for i, r in enumerate(qrows):
            same = torch.zeros(n, dtype=torch.bool, device="cuda")
            for t0 in range(0, T, 100):
                part = sig[t0:t0 + 100]
                same |= (part == part[:, r:r + 1, :]).all(dim=2).any(dim=0)
            exp = torch.nonzero(same).flatten().cpu().numpy().astype(np.int32)
            lo, hi = int(got["offsets"][i]), int(got["offsets"][i + 1])
            assert hi - lo == exp.size and r in exp
            np.testing.assert_array_equal(got["indices"][lo:hi], exp)
    finally:
        if ch:
            lib.culsh_candidates_free(ch)
        lib.culsh_index_free(ih)


def test_item_count_of_2_31_is_refused(ctx):
    """One row more than the limit: refused before any device work (the rows are never read)."""
    import ctypes as C

    from culsh_amd import _lib as L
    from culsh_amd.abi import dev, hp, ptr

    _announce("items_2_31_refused")
    T, H, d = 1024, 4, 8
    n = (1 << 31) // T                                       # n * T = 2^31 exactly
    tiny = dev(np.zeros((4, d), dtype=np.float32))           # stands for X: the call must not touch it
    P = np.zeros((T * H, d), dtype=np.float32)
    ih = C.c_void_p()
    status = ctx.lib.culsh_rplsh_fit_f32(ctx.h, ptr(tiny), n, d, T, H, 1, hp(P), C.byref(ih))
    assert status == L.ERR_LIMIT and not ih.value
    assert b"2^31" in ctx.lib.culsh_last_error()


def test_config5_full_size_invariants(ctx):
    """Benchmark configuration 5 of the reference at its real shape (4M x 768 rows of a 1000-component Gaussian mixture on the
    unit sphere, 64 tables x 16 hashes), 20k queries in batches of 10k: the index takes 2^28 items, a
    query four bitmap passes over the row range, and the batches are merged.  Data are made and the
    properties checked on the device; a sample of buckets and of queries is compared with brute force."""
    _announce("config5_full_size")
    import ctypes as C

    import torch
    from abi import hp, ptr
    from culsh_amd import _lib as L

    n, d, nq, T, H, batch = 4_000_000, 768, 20_000, 64, 16, 10_000
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    centres = torch.randn(1000, d, device="cuda", generator=g)

    def mixture(rows):
        out = torch.empty(rows, d, device="cuda", dtype=torch.float32)
        for s0 in range(0, rows, 500_000):
            m = min(500_000, rows - s0)
            comp = torch.randint(0, 1000, (m,), device="cuda", generator=g)
            x = centres[comp] + 0.3 * torch.randn(m, d, device="cuda", generator=g)
            out[s0:s0 + m] = x / x.norm(dim=1, keepdim=True)
        return out

    X, Q = mixture(n), mixture(nq)
    P = torch.randn(T * H, d, device="cuda", generator=g)
    P_host = np.ascontiguousarray(P.cpu().numpy())
    torch.cuda.synchronize()
    ih = C.c_void_p()
    L.check(ctx.lib.culsh_rplsh_fit_f32(ctx.h, ptr(X), n, d, T, H, 42, hp(P_host), C.byref(ih)))
    ix = ctx.index_arrays(ih)
    N = n * T
    B = int(ix["n_total_buckets"])
    tbo = torch.from_numpy(ix["table_bucket_offsets"].astype(np.int64)).cuda()
    bco = torch.from_numpy(ix["bucket_candidate_offsets"].astype(np.int64)).cuda()
    cand = torch.from_numpy(ix["all_candidate_indices"]).cuda()
    assert tbo[0] == 0 and tbo[-1] == B and bool((tbo.diff() > 0).all())
    assert bco[0] == 0 and bco[-1] == N and bool((bco.diff() > 0).all())
    assert bool((bco[tbo[:-1]] == torch.arange(T, device="cuda") * n).all())   # a table's first bucket starts its segment
    for t in range(T):                                                          # every table holds every row once
        assert bool((torch.bincount(cand[t * n:(t + 1) * n], minlength=n) == 1).all()), t
    descents = torch.nonzero(cand[1:] < cand[:-1]).flatten() + 1                # rows ascend inside a bucket
    assert bool(torch.isin(descents, bco).all())
    sig = torch.from_numpy(ix["all_bucket_signatures"].reshape(B, H)).cuda().to(torch.int64)
    keys = (sig * (1 << torch.arange(H - 1, -1, -1, device="cuda"))).sum(1)     # 16 sign bytes as a number
    inc = keys.diff() > 0
    inc[tbo[1:-1] - 1] = True                                                   # table boundaries may descend
    assert bool(inc.all())
    # a bucket's signature is the sign pattern of the rows in it (float64 projection, outside the band)
    pos = torch.arange(0, N, 100_003, device="cuda")
    b = torch.searchsorted(bco, pos, right=True) - 1
    rows, tt, k = cand[pos].long(), pos // n, torch.arange(len(pos), device="cuda")
    proj = (X[rows].double() @ P.double().T).view(-1, T, H)[k, tt]
    scale = (X[rows].abs().double() @ P.abs().double().T).view(-1, T, H)[k, tt]
    assert int((((proj >= 0).to(torch.int64) != sig[b]) & (proj.abs() > TOL * scale)).sum()) == 0
    # queries
    ch = C.c_void_p()
    L.check(ctx.lib.culsh_rplsh_query_f32(ctx.h, ptr(Q), nq, ih, batch, C.byref(ch)))
    got = ctx.candidates_arrays(ch)
    off = torch.from_numpy(got["offsets"].astype(np.int64)).cuda()
    idx = torch.from_numpy(got["indices"]).cuda()
    assert off[0] == 0 and int(off[-1]) == len(idx) and bool((off.diff() >= 0).all())
    assert np.array_equal(np.diff(got["offsets"].astype(np.int64)), got["counts"].astype(np.int64))
    inside = torch.ones(len(idx), dtype=torch.bool, device="cuda")
    starts = off[1:-1]
    inside[starts[starts < len(idx)]] = False                                   # first element of the next query
    assert bool(((idx[1:] > idx[:-1]) | ~inside[1:]).all())                     # ascending, duplicate-free per query
    assert int(idx.min()) >= 0 and int(idx.max()) < n
    sample = [0, 9_999, 10_000, 14_321, 19_999]                                 # both batches and their edges
    qsig = ctx.rplsh_hash(Q[sample].cpu().numpy(), P_host, T, H)                # [T][5][H]
    sig_np = ix["all_bucket_signatures"].reshape(B, H)
    tbo_np, bco_np, cand_np = ix["table_bucket_offsets"], ix["bucket_candidate_offsets"], ix["all_candidate_indices"]
    for j, q in enumerate(sample):
        exp = []
        for t in range(T):
            lo, hi = tbo_np[t], tbo_np[t + 1]
            hit = np.flatnonzero((sig_np[lo:hi] == qsig[t, j]).all(axis=1))
            if len(hit):
                bb = lo + hit[0]
                exp.append(cand_np[bco_np[bb]:bco_np[bb + 1]])
        exp = np.unique(np.concatenate(exp)) if exp else np.zeros(0, np.int32)
        np.testing.assert_array_equal(got["indices"][int(got["offsets"][q]):int(got["offsets"][q + 1])], exp)
    ctx.free_index(ih)
    del X, Q, cand, sig, idx
    torch.cuda.empty_cache()
    ctx.lib.culsh_memory_trim()


@pytest.mark.parametrize("first_seed", [0, 12, 24])
def test_random_shapes_all_families(ctx, first_seed):
    """Twelve seeded draws per case of (family, rows, queries, tables, hashes, features, dtype, batch
    size) from lists that sit on and around the tile sizes of the kernels: index, candidates (batched
    or not) and fit_query against the oracle given the GPU's own signatures."""
    from abi import assert_candidates_match, assert_index_matches

    for s in range(first_seed, first_seed + 12):
        rng = np.random.default_rng(s)
        fam = ["rplsh", "pslsh", "minhash"][s % 3]
        n = int(rng.choice([1, 2, 63, 64, 65, 127, 128, 129, 1000, 4095, 4096, 4097, 8191, 8192, 8193, 12345, 20000]))
        nq = int(rng.choice([1, 3, 64, 100, 257]))
        T = int(rng.choice([1, 2, 3, 7, 16, 33, 70]))
        H = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 17, 32, 33, 40]))
        d = int(rng.choice([1, 3, 4, 15, 16, 17, 64, 100, 128, 130]))
        dtype = np.float32 if rng.random() < 0.7 else np.float64
        bs = int(rng.choice([-1, 1, 10, 64]))
        _announce("random_shapes", s, fam, n, nq, T, H, d, dtype.__name__, bs)
        if fam == "minhash":
            dcols = int(rng.choice([5, 50, 400, 70000]))
            nnz = int(rng.choice([1, 4, 30]))
            indices, indptr = make_csr(rng, n, dcols, nnz, empty_rows=(0,) if n > 3 and rng.random() < 0.5 else ())
            qindices, qindptr = make_csr(rng, nq, dcols, nnz)
            A, B = o.generate_hash_integers(s, T * H)
            sig = o.minhash_hash(indices, indptr, A, B, T, H)
            qsig = o.minhash_hash(qindices, qindptr, A, B, T, H)
            ih = ctx.minhash_fit(indices, indptr, dcols, T, H, A=A, B=B)
            got_q = ctx.minhash_query(qindices, qindptr, ih)
            got_fq = ctx.minhash_fit_query(indices, indptr, dcols, T, H, A=A, B=B)
        else:
            X = rng.standard_normal((n, d)).astype(dtype)
            Q = np.concatenate([X[:min(n, nq // 2 + 1)], rng.standard_normal((nq, d)).astype(dtype)])[:nq]
            if fam == "rplsh":
                P = rng.standard_normal((T * H, d)).astype(dtype)
                sig, qsig = ctx.rplsh_hash(X, P, T, H), ctx.rplsh_hash(Q, P, T, H)
                ih = ctx.rplsh_fit(X, T, H, P=P)
                got_q = ctx.rplsh_query(Q, ih, batch_size=bs)
                got_fq = ctx.rplsh_fit_query(X, T, H, P=P)
            else:
                w = int(rng.choice([1, 2, 4, 50]))
                P, b = o.generate_random_projections_biases(s, T * H, d, w, dtype)
                sig, qsig = ctx.pslsh_hash(X, P, b, T, H), ctx.pslsh_hash(Q, P, b, T, H)
                ih = ctx.pslsh_fit(X, T, H, w, P=P, b=b)
                got_q = ctx.pslsh_query(Q, ih, batch_size=bs)
                got_fq = ctx.pslsh_fit_query(X, T, H, w, P=P, b=b)
        exp_ix = o.fit_index(sig, H)
        assert_index_matches(ctx.index_arrays(ih), exp_ix)
        assert_candidates_match(got_q, o.query_index(qsig, exp_ix))
        assert_candidates_match(got_fq, o.fit_query(sig, H))
        ctx.free_index(ih)


def test_objects_cross_contexts(ctx):
    """An index built through one context answers queries issued through another (objects belong to
    the device, not to the context that made them), also after the first context is gone, and two
    contexts used in turns do not disturb each other's scratch memory."""
    _announce("cross_contexts")
    from abi import Ctx, assert_candidates_match

    rng = np.random.default_rng(11)
    T, n, nq, H = 5, 6000, 120, 3
    sig = random_sigs(rng, T, n, H, "rplsh")
    qsig = random_sigs(rng, T, nq, H, "rplsh")
    exp = o.query_index(qsig, o.fit_index(sig, H))
    other = Ctx(0)
    ih, _ = other.core_fit_index(sig, H)
    assert_candidates_match(ctx.core_query_index(qsig, ih), exp)        # built there, queried here
    ih2, _ = ctx.core_fit_index(sig, H)
    for _ in range(3):                                                    # in turns
        assert_candidates_match(other.core_query_index(qsig, ih2), exp)
        assert_candidates_match(ctx.core_query_index(qsig, ih), exp)
    other.close()
    assert_candidates_match(ctx.core_query_index(qsig, ih), exp)        # its maker is gone
    ctx.free_index(ih)
    ctx.free_index(ih2)


def test_contexts_on_host_threads(c_oracle):
    """One context per host thread: four threads fit and query at the same time (ctypes releases the
    interpreter lock during a call, so the library's calls, the block cache and the kernels with
    their waits between workgroups really overlap), each on its own data and several times over, and
    every result is the oracle's."""
    _announce("contexts_on_host_threads")
    import threading
    from abi import Ctx, assert_candidates_match, assert_index_matches

    shapes = [(4, 70000, 300, 2), (6, 9000, 200, 3), (2, 150000, 64, 2), (33, 3000, 100, 4)]  # T, n, nq, H
    cases = []
    for i, (T, n, nq, H) in enumerate(shapes):
        rng = np.random.default_rng(500 + i)
        sig = random_sigs(rng, T, n, H, "rplsh")
        qsig = random_sigs(rng, T, nq, H, "rplsh")
        cix = c_oracle.fit_index_c(sig, H)
        cases.append((sig, qsig, H, n, cix.to_numpy(n), c_oracle.query_index_c(qsig, cix)))
    failures = []
    start = threading.Barrier(len(cases))

    def work(case):
        sig, qsig, H, n, exp_ix, exp_cand = case
        try:
            c = Ctx(0)
            start.wait(timeout=60)
            for _ in range(6):
                ih, _ = c.core_fit_index(sig, H)
                assert_index_matches(c.index_arrays(ih), exp_ix)
                assert_candidates_match(c.core_query_index(qsig, ih), exp_cand)
                c.free_index(ih)
            c.close()
        except BaseException as e:  # reported by the main thread
            failures.append(repr(e))

    threads = [threading.Thread(target=work, args=(case,)) for case in cases]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not failures, failures


def test_minhash_rank_keys_edge_cases(ctx):
    """MinHash keys are stored as column ranks when every fitted column id is below n_features.
    Checked against the oracle: query rows whose minimum comes from a column >= n_features (they
    can match nothing in that table), empty rows on both sides, queries given as raw signatures
    through the stage-level call, and a fit that contains an out-of-range column (plain keys)."""
    _announce("minhash_rank_edges")
    rng = np.random.default_rng(31)
    n, d, T, H, nq = 3000, 400, 6, 3, 200
    indices, indptr = make_csr(rng, n, d, 6, empty_rows=(1, 2, 50))
    A, B = o.generate_hash_integers(5, T * H)
    qrows = []
    for i in range(nq):
        r = indices[indptr[i]:indptr[i + 1]].astype(np.int64)
        if i % 5 == 0:
            r = np.concatenate([r, rng.integers(d, d + 4000, size=2)])   # columns the fit never saw
        if i % 17 == 0:
            r = np.zeros(0, dtype=np.int64)
        qrows.append(np.unique(r))
    qindptr = np.concatenate([[0], np.cumsum([len(r) for r in qrows])]).astype(np.int32)
    qindices = np.concatenate(qrows).astype(np.int32)
    from abi import assert_candidates_match, assert_index_matches

    sig = o.minhash_hash(indices, indptr, A, B, T, H)
    qsig = o.minhash_hash(qindices, qindptr, A, B, T, H)
    exp_ix = o.fit_index(sig, H)
    exp = o.query_index(qsig, exp_ix)
    ih = ctx.minhash_fit(indices, indptr, d, T, H, A=A, B=B)
    assert_index_matches(ctx.index_arrays(ih), exp_ix)
    assert_candidates_match(ctx.minhash_query(qindices, qindptr, ih), exp)
    assert_candidates_match(ctx.core_query_index(qsig, ih), exp)          # raw signatures -> rank keys
    np.testing.assert_array_equal(ctx.core_find_matching_buckets(qsig, ih), o.find_matching_buckets_fast(qsig, exp_ix))
    ctx.free_index(ih)
    # multipliers that are 0 modulo the prime (every column hashes alike), at and above the prime, and
    # offsets at and above it: the column of the minimum is still the one the reference's scan keeps
    A3, B3 = A.copy(), B.copy()
    A3[0], A3[1], A3[2], A3[3] = 0, 4294967291, 4294967295, 1
    B3[0], B3[2], B3[4] = 4294967295, 4294967291, 0
    sig3 = o.minhash_hash(indices, indptr, A3, B3, T, H)
    ih3 = ctx.minhash_fit(indices, indptr, d, T, H, A=A3, B=B3)
    exp_ix3 = o.fit_index(sig3, H)
    assert_index_matches(ctx.index_arrays(ih3), exp_ix3)
    qsig3 = o.minhash_hash(qindices, qindptr, A3, B3, T, H)
    assert_candidates_match(ctx.minhash_query(qindices, qindptr, ih3), o.query_index(qsig3, exp_ix3))
    ctx.free_index(ih3)
    # a fitted row with a column id >= n_features: every id is hashed as it is (minhash/hash.cuh:97-104)
    # (the rank kernel flags it and the fit is repeated with plain keys); ids next to the bound, beyond
    # the range of the cheaper hash, at the top of int32, and in the last row
    for pos, bad_id in ((7, d + 123), (0, d), (len(indices) - 1, (1 << 25) + 5), (indptr[n // 2], (1 << 31) - 1)):
        bad = indices.copy()
        bad[pos] = bad_id
        sig2 = o.minhash_hash(bad, indptr, A, B, T, H)
        ih2 = ctx.minhash_fit(bad, indptr, d, T, H, A=A, B=B)
        exp_ix2 = o.fit_index(sig2, H)
        assert_index_matches(ctx.index_arrays(ih2), exp_ix2)
        assert_candidates_match(ctx.minhash_query(qindices, qindptr, ih2), o.query_index(qsig, exp_ix2))
        ctx.free_index(ih2)
    bad = indices.copy()
    bad[11] = d + 1
    assert_candidates_match(ctx.minhash_fit_query(bad, indptr, d, T, H, A=A, B=B),
                            o.fit_query(o.minhash_hash(bad, indptr, A, B, T, H), H))
    # and a fit with rank keys straight after one that fell back: the flag does not stick
    ih4 = ctx.minhash_fit(indices, indptr, d, T, H, A=A, B=B)
    assert_index_matches(ctx.index_arrays(ih4), exp_ix)
    ctx.free_index(ih4)
