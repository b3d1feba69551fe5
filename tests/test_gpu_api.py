"""
GPU tests of the public Python API (culsh_amd.RPLSH / PStableLSH / MinHashLSH), written
after the reference's own test-suite (python/tests/test_rplsh.py, test_pslsh.py,
test_minhash.py): recall against a CPU LSH with independent random parameters, save/load
round trips, fit_query == fit + query, batched == unbatched, auto window size.
"""

import os

import numpy as np
import pytest
import scipy.sparse

from oracle import culsh_oracle as o

pytestmark = pytest.mark.gpu


def dense(n, d, dtype, seed=42):
    return np.random.default_rng(seed).standard_normal((n, d)).astype(dtype)


def sparse(n, d, density, seed=42):
    rs = np.random.RandomState(seed)
    X = scipy.sparse.random(n, d, density=density, format="csr", dtype=np.float32, random_state=rs)
    X.data[:] = 1.0
    X.indices = X.indices.astype(np.int32)
    X.indptr = X.indptr.astype(np.int32)
    return X


def recall_at_k(X, n_eval, k, indices, offsets, topk):
    rec = []
    for q in range(n_eval):
        got = indices[int(offsets[q]):int(offsets[q + 1])]
        rec.append(len(np.intersect1d(got, topk(q))) / k)
    return float(np.mean(rec))


def oracle_recall(sig, n_eval, k, H, topk):
    c = o.query_index(sig[:, :n_eval], o.fit_index(sig, H))
    return recall_at_k(None, n_eval, k, c.query_candidate_indices, c.query_candidate_offsets, topk)


# ---------------------------------------------------------------- RPLSH
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n_hash_tables", [8, 32, 64])
@pytest.mark.parametrize("n_hashes", [8, 16])
def test_rplsh_recall_vs_cpu_lsh(dtype, n_hash_tables, n_hashes):
    """python/tests/test_rplsh.py:27-73: mean recall@20 of 50 self-queries within 0.05 of a
    CPU LSH that draws its own projections."""
    from culsh_amd import RPLSH

    n, d, n_eval, k = 1000, 100, 50, 20
    X = dense(n, d, dtype)
    Xn = X / np.linalg.norm(X, axis=1, keepdims=True)

    def topk(q):
        return np.argsort(Xn @ Xn[q])[-k:]

    P = np.random.default_rng(7).standard_normal((n_hash_tables * n_hashes, d)).astype(dtype)
    ref = oracle_recall(o.rplsh_hash(X, P, n_hash_tables, n_hashes), n_eval, k, n_hashes, topk)
    cand = RPLSH(n_hash_tables=n_hash_tables, n_hashes=n_hashes, seed=42).fit_query(X)
    got = recall_at_k(X, n_eval, k, cand.get_indices(), cand.get_offsets(), topk)
    assert abs(got - ref) < 0.05 and got <= 1.0
    assert cand.n_queries == n and cand.get_counts().dtype == np.uint64


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("as_torch", [False, True])
def test_rplsh_save_load(tmp_path, dtype, as_torch):
    """python/tests/test_rplsh.py:76-142"""
    import torch

    from culsh_amd import RPLSH, RPLSHModel

    X = dense(1000, 64, dtype)
    Xin = torch.from_numpy(X).cuda() if as_torch else X
    model = RPLSH(n_hash_tables=16, n_hashes=8, seed=42).fit(Xin)
    path = os.path.join(tmp_path, "rplsh_model.npz")
    model.save(path)
    loaded = RPLSHModel.load(path)
    assert (loaded.n_hash_tables, loaded.n_hashes, loaded.n_features) == (16, 8, 64)
    for attr in ("n_total_candidates", "n_total_buckets", "n_hash_tables", "n_hashes", "sig_nbytes", "n_features",
                 "seed", "is_double"):
        assert getattr(loaded.index, attr) == getattr(model.index, attr), attr
    assert model.index.sig_nbytes == 8 and model.index.is_double == (dtype == np.float64)
    for getter in ("get_candidate_indices", "get_bucket_signatures", "get_bucket_candidate_offsets",
                   "get_table_bucket_offsets", "get_projection_matrix"):
        np.testing.assert_array_equal(getattr(loaded.index, getter)(), getattr(model.index, getter)())
    assert set(np.unique(model.index.get_bucket_signatures())) <= {0, 1}
    assert model.index.size_bytes() == loaded.index.size_bytes() > 0
    a, b = model.query(Xin[:100]), loaded.query(Xin[:100])
    np.testing.assert_array_equal(a.get_indices(), b.get_indices())
    np.testing.assert_array_equal(a.get_offsets(), b.get_offsets())
    data = np.load(path)
    assert sorted(data.files) == sorted([
        "n_hash_tables", "n_hashes", "n_features", "n_total_candidates", "n_total_buckets", "seed", "sig_nbytes",
        "is_double", "candidate_indices", "bucket_signatures", "bucket_candidate_offsets", "table_bucket_offsets",
        "projection"])


def test_load_refuses_arrays_that_do_not_add_up():
    """Offsets that decrease or do not span their arrays, and candidate indices beyond the row count,
    would send the query kernels outside the arrays; loading such an index is an error (the
    reference loads it unchecked)."""
    from culsh_amd import RPLSH
    from culsh_amd._culsh_core import RPLSHIndex

    X = dense(500, 32, np.float32)
    ix = RPLSH(n_hash_tables=4, n_hashes=6, seed=3).fit(X).index
    good = dict(candidate_indices=ix.get_candidate_indices(), bucket_signatures=ix.get_bucket_signatures(),
                bucket_candidate_offsets=ix.get_bucket_candidate_offsets(),
                table_bucket_offsets=ix.get_table_bucket_offsets(), projection=ix.get_projection_matrix(),
                n_total_candidates=ix.n_total_candidates, n_total_buckets=ix.n_total_buckets,
                n_hash_tables=ix.n_hash_tables, n_hashes=ix.n_hashes, sig_nbytes=ix.sig_nbytes,
                n_features=ix.n_features, seed=ix.seed)
    again = RPLSHIndex.load_float(**good)
    np.testing.assert_array_equal(again.get_candidate_indices(), good["candidate_indices"])

    def broken(name, change):
        bad = dict(good)
        arr = good[name].copy()
        change(arr)
        bad[name] = arr
        with pytest.raises(RuntimeError):
            RPLSHIndex.load_float(**bad)

    broken("candidate_indices", lambda a: a.__setitem__(7, 500))          # one past the last row
    broken("candidate_indices", lambda a: a.__setitem__(0, -1))
    broken("bucket_candidate_offsets", lambda a: a.__setitem__(3, a[4] + 1))   # decreases afterwards
    broken("bucket_candidate_offsets", lambda a: a.__setitem__(-1, a[-1] + 5))  # beyond the candidates
    broken("table_bucket_offsets", lambda a: a.__setitem__(2, a[1] - 1))
    broken("table_bucket_offsets", lambda a: a.__setitem__(0, 1))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_rplsh_fit_query_equals_fit_then_query(dtype):
    """python/tests/test_rplsh.py:145-174"""
    from culsh_amd import RPLSH

    X = dense(1000, 64, dtype)
    lsh = RPLSH(n_hash_tables=16, n_hashes=8, seed=42)
    a = lsh.fit_query(X)
    b = lsh.fit(X).query(X)
    np.testing.assert_array_equal(a.get_indices(), b.get_indices())
    np.testing.assert_array_equal(a.get_offsets(), b.get_offsets())
    c = lsh.fit_query(X, batch_size=300)      # falls back to fit + batched query
    np.testing.assert_array_equal(a.get_indices(), c.get_indices())


def test_estimator_fitted_again_matches_fresh_estimators():
    """An estimator keeps its core (stream, scratch, seeded parameters) between fits: fitting it on
    other data, another shape and another dtype gives what a fresh estimator gives, and models
    fitted earlier keep answering from their own index."""
    from culsh_amd import RPLSH, PStableLSH

    lsh = RPLSH(n_hash_tables=8, n_hashes=8, seed=7)
    inputs = [dense(500, 32, np.float32, seed=1), dense(700, 48, np.float32, seed=2), dense(300, 32, np.float64, seed=3)]
    models = [lsh.fit(X) for X in inputs]
    for X, model in zip(inputs, models):
        fresh = RPLSH(n_hash_tables=8, n_hashes=8, seed=7).fit(X)
        a, b = model.query(X[:50]), fresh.query(X[:50])
        np.testing.assert_array_equal(a.get_indices(), b.get_indices())
        np.testing.assert_array_equal(a.get_offsets(), b.get_offsets())
        np.testing.assert_array_equal(model.index.get_projection_matrix(), fresh.index.get_projection_matrix())
    ps = PStableLSH(n_hash_tables=4, n_hashes=4, window_size="auto", seed=3)   # the window, hence the core, follows the data
    for X in (inputs[0], 10.0 * inputs[0]):
        a = ps.fit(X).query(X[:20])
        b = PStableLSH(n_hash_tables=4, n_hashes=4, window_size="auto", seed=3).fit(X).query(X[:20])
        np.testing.assert_array_equal(a.get_indices(), b.get_indices())


@pytest.mark.parametrize("batch_size", [10, 50, 100])
def test_rplsh_batched_query(batch_size):
    """python/tests/test_rplsh.py:177-209"""
    from culsh_amd import RPLSH

    X, Q = dense(1000, 64, np.float32), dense(100, 64, np.float32, seed=1)
    model = RPLSH(n_hash_tables=16, n_hashes=8, seed=42).fit(X)
    a, b = model.query(Q), model.query(Q, batch_size=batch_size)
    np.testing.assert_array_equal(a.get_indices(), b.get_indices())
    np.testing.assert_array_equal(a.get_offsets(), b.get_offsets())
    np.testing.assert_array_equal(a.get_counts(), b.get_counts())


def test_rplsh_errors_and_device_getters():
    import torch

    from culsh_amd import RPLSH

    X = dense(500, 32, np.float32)
    model = RPLSH(4, 4, seed=1).fit(X)
    with pytest.raises(ValueError, match=r"Query features \(16\) != fitted features \(32\)"):
        model.query(dense(10, 16, np.float32))
    with pytest.raises(TypeError, match="Unsupported dtype"):
        model.query(X.astype(np.float16))
    with pytest.raises(TypeError, match="Unsupported dtype"):
        RPLSH(4, 4).fit(X.astype(np.int32))
    with pytest.raises(RuntimeError, match="fitted with float32, but query is float64"):
        model.query(X.astype(np.float64))
    with pytest.raises(ValueError, match="Expected 2D array"):
        model.query(X[0])
    c = model.query(X[:20])
    t = c.get_indices(as_torch=True)
    assert t.is_cuda and t.dtype == torch.int32
    np.testing.assert_array_equal(t.cpu().numpy(), c.get_indices())
    np.testing.assert_array_equal(c.get_offsets(as_torch=True).cpu().numpy().view(np.uint64), c.get_offsets())
    assert not c.empty() and c.n_total_candidates == len(c.get_indices())
    # non-contiguous input is made contiguous
    Xt = torch.from_numpy(np.ascontiguousarray(X.T)).cuda().T
    assert not Xt.is_contiguous()
    np.testing.assert_array_equal(RPLSH(4, 4, seed=1).fit(Xt).index.get_candidate_indices(),
                                  model.index.get_candidate_indices())


# ---------------------------------------------------------------- p-stable
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("window_size", [4, 8])
def test_pslsh_recall_vs_cpu_lsh(dtype, window_size):
    """python/tests/test_pslsh.py:26-85"""
    from culsh_amd import PStableLSH

    n, d, n_eval, k, T, H = 1000, 100, 50, 20, 32, 4
    X = dense(n, d, dtype)

    def topk(q):
        return np.argsort(np.linalg.norm(X - X[q], axis=1))[:k]

    rng = np.random.default_rng(7)
    P = (rng.standard_normal((T * H, d)) / window_size).astype(dtype)
    b = rng.uniform(0, 1, size=T * H).astype(dtype)
    ref = oracle_recall(o.pslsh_hash(X, P, b, T, H), n_eval, k, H, topk)
    cand = PStableLSH(n_hash_tables=T, n_hashes=H, window_size=window_size, seed=42).fit_query(X)
    got = recall_at_k(X, n_eval, k, cand.get_indices(), cand.get_offsets(), topk)
    assert abs(got - ref) < 0.05 and got <= 1.0


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pslsh_save_load_fit_query_batched(tmp_path, dtype):
    """python/tests/test_pslsh.py:88-240"""
    from culsh_amd import PStableLSH, PStableLSHModel

    X = dense(1000, 64, dtype)
    lsh = PStableLSH(n_hash_tables=16, n_hashes=4, window_size=4, seed=42)
    model = lsh.fit(X)
    path = os.path.join(tmp_path, "pslsh_model.npz")
    model.save(path)
    loaded = PStableLSHModel.load(path)
    assert loaded.window_size == 4 and model.index.sig_nbytes == 16
    for getter in ("get_candidate_indices", "get_bucket_signatures", "get_bucket_candidate_offsets",
                   "get_table_bucket_offsets", "get_projection_matrix", "get_bias"):
        np.testing.assert_array_equal(getattr(loaded.index, getter)(), getattr(model.index, getter)())
    bias = model.index.get_bias()
    assert bias.dtype == dtype and bias.min() > 0 and bias.max() <= 1
    a, b = model.query(X[:100]), loaded.query(X[:100])
    np.testing.assert_array_equal(a.get_indices(), b.get_indices())
    fq = lsh.fit_query(X)
    full = model.query(X)
    np.testing.assert_array_equal(fq.get_indices(), full.get_indices())
    np.testing.assert_array_equal(fq.get_offsets(), full.get_offsets())
    for bs in (10, 50, 100):
        c = model.query(X[:100], batch_size=bs)
        np.testing.assert_array_equal(a.get_indices(), c.get_indices())
        np.testing.assert_array_equal(a.get_offsets(), c.get_offsets())
    assert "window_size" in np.load(path).files and "bias" in np.load(path).files


def test_pslsh_auto_window_size():
    """python/tests/test_pslsh.py:243-255"""
    import torch

    from culsh_amd import PStableLSH

    X = dense(1000, 32, np.float32)
    X = (100.0 * X / np.linalg.norm(X, axis=1, keepdims=True)).astype(np.float32)
    assert PStableLSH._estimate_window_size(torch.from_numpy(X).cuda()) in (99, 100)
    model = PStableLSH(n_hash_tables=4, n_hashes=2, window_size="auto", seed=3).fit(X)
    assert model.window_size in (99, 100)


# ---------------------------------------------------------------- MinHash
@pytest.mark.parametrize("density", [0.1, 0.5])
def test_minhash_recall_vs_cpu_lsh(density):
    """python/tests/test_minhash.py:36-82"""
    from culsh_amd import MinHashLSH

    n, d, n_eval, k, T, H = 1000, 100, 50, 20, 32, 2
    X = sparse(n, d, density)
    Xd = (X.toarray() > 0)

    def topk(q):
        inter = (Xd & Xd[q]).sum(1)
        union = (Xd | Xd[q]).sum(1)
        return np.argsort(inter / np.maximum(union, 1))[-k:]

    A, B = o.generate_hash_integers(7, T * H)
    ref = oracle_recall(o.minhash_hash(X.indices, X.indptr, A, B, T, H), n_eval, k, H, topk)
    cand = MinHashLSH(n_hash_tables=T, n_hashes=H, seed=42).fit_query(X)
    got = recall_at_k(X, n_eval, k, cand.get_indices(), cand.get_offsets(), topk)
    assert abs(got - ref) < 0.05 and got <= 1.0


def test_minhash_save_load_and_fit_query(tmp_path):
    """python/tests/test_minhash.py:85-183"""
    from culsh_amd import MinHashLSH, MinHashLSHModel

    X = sparse(1000, 200, 0.05)
    lsh = MinHashLSH(n_hash_tables=16, n_hashes=4, seed=42)
    model = lsh.fit(X)
    path = os.path.join(tmp_path, "minhash_model.npz")
    model.save(path)
    loaded = MinHashLSHModel.load(path)
    for getter in ("get_candidate_indices", "get_bucket_signatures", "get_bucket_candidate_offsets",
                   "get_table_bucket_offsets", "get_hash_a", "get_hash_b"):
        np.testing.assert_array_equal(getattr(loaded.index, getter)(), getattr(model.index, getter)())
    assert model.index.sig_nbytes == 16 and model.index.get_hash_a().dtype == np.uint32
    a, b = model.query(X[:100]), loaded.query(X[:100])
    np.testing.assert_array_equal(a.get_indices(), b.get_indices())
    fq, full = lsh.fit_query(X), model.query(X)
    np.testing.assert_array_equal(fq.get_indices(), full.get_indices())
    np.testing.assert_array_equal(fq.get_offsets(), full.get_offsets())
    # signatures follow the documented definition for the seeded coefficients
    A, B = model.index.get_hash_a(), model.index.get_hash_b()
    exp = o.fit_index(o.minhash_hash(X.indices, X.indptr, A, B, 16, 4), 4)
    np.testing.assert_array_equal(model.index.get_candidate_indices(), exp.all_candidate_indices)
    np.testing.assert_array_equal(model.index.get_bucket_signatures(), exp.all_bucket_signatures)
    X64 = X.copy()
    X64.indices = X64.indices.astype(np.int64)
    with pytest.raises(ValueError, match="requires int32 indices"):
        lsh.fit(X64)


def test_minhash_prime_is_a_parameter(tmp_path):
    """`prime` (not in the reference, whose prime is fixed at 2^32 - 5, minhash/hash.cuh:17): a model fitted
    modulo 2^31 - 1 follows the definition with that prime, names it in its file and comes back from the
    file as it was; a default model's file holds the reference's keys only."""
    from culsh_amd import MinHashLSH, MinHashLSHModel

    p31 = o.MINHASH_PRIME_MERSENNE
    X = sparse(1500, 300, 0.05)
    T, H = 8, 3
    with pytest.raises(ValueError, match="prime"):
        MinHashLSH(n_hash_tables=T, n_hashes=H, seed=3, prime=4294967295)
    lsh = MinHashLSH(n_hash_tables=T, n_hashes=H, seed=3, prime=p31)
    model = lsh.fit(X)
    assert lsh.prime == p31 and model.prime == p31 and model.index.prime == p31
    A, B = model.index.get_hash_a(), model.index.get_hash_b()
    np.testing.assert_array_equal(A, o.generate_hash_integers(3, T * H, p31)[0])
    exp = o.fit_index(o.minhash_hash(X.indices, X.indptr, A, B, T, H, p31), H)
    np.testing.assert_array_equal(model.index.get_candidate_indices(), exp.all_candidate_indices)
    np.testing.assert_array_equal(model.index.get_bucket_signatures(), exp.all_bucket_signatures)
    want = o.query_index(o.minhash_hash(X.indices, X.indptr, A, B, T, H, p31)[:, :200], exp)
    got = model.query(X[:200])
    np.testing.assert_array_equal(got.get_indices(), want.query_candidate_indices)
    np.testing.assert_array_equal(got.get_offsets(), want.query_candidate_offsets)
    path = os.path.join(tmp_path, "minhash_p31.npz")
    model.save(path)
    assert int(np.load(path)["prime"]) == p31
    loaded = MinHashLSHModel.load(path)
    assert loaded.prime == p31 and _key_form(loaded.index) == _key_form(model.index)
    again = loaded.query(X[:200])
    np.testing.assert_array_equal(again.get_indices(), got.get_indices())
    np.testing.assert_array_equal(again.get_offsets(), got.get_offsets())
    fq = lsh.fit_query(X)
    full = model.query(X)
    np.testing.assert_array_equal(fq.get_indices(), full.get_indices())
    # the default: the reference's prime, and no key beyond the reference's in the file
    plain = MinHashLSH(n_hash_tables=T, n_hashes=H, seed=3).fit(X)
    assert plain.prime == o.MINHASH_PRIME
    path2 = os.path.join(tmp_path, "minhash_default.npz")
    plain.save(path2)
    assert "prime" not in np.load(path2).files
    assert MinHashLSHModel.load(path2).prime == o.MINHASH_PRIME


def _key_form(index):
    """(key words per bucket, encoding) of an index object of the extension-module surface."""
    import ctypes as C

    w, enc = C.c_int32(), C.c_int32()
    from culsh_amd import _lib as L

    L.check(index._lib.culsh_index_key_form(index._h, C.byref(w), C.byref(enc)))
    return w.value, enc.value


def test_loaded_models_look_buckets_up_like_fitted_ones(tmp_path):
    """A model that comes back from `load` runs the same bucket lookup as the one `fit` returned: the
    loaded index has the fitted index's key form (p-stable hashes as ranks of the values seen at fit
    time, 8 words -> 2; MinHash values as ranks of their columns, 4 words -> 2; RPLSH one bit per hash)
    and returns the same candidates, also for queries whose hashes no fitted row has.  A MinHash model
    fitted on column ids at or beyond n_features keeps plain keys on both sides."""
    from culsh_amd import MinHashLSH, MinHashLSHModel, PStableLSH, PStableLSHModel, RPLSH, RPLSHModel

    X = dense(3000, 32, np.float32, seed=11)
    Q = np.concatenate([X[:150], 40.0 * dense(50, 32, np.float32, seed=12)])     # far-away queries: unseen hash values
    for est, cls, words, enc in ((PStableLSH(n_hash_tables=6, n_hashes=8, window_size=4, seed=3), PStableLSHModel, 2, 2),
                                 (RPLSH(n_hash_tables=6, n_hashes=40, seed=3), RPLSHModel, 2, 1)):
        model = est.fit(X)
        path = os.path.join(tmp_path, cls.__name__ + ".npz")
        model.save(path)
        loaded = cls.load(path)
        assert _key_form(model.index) == _key_form(loaded.index)
        assert _key_form(model.index)[1] == enc and _key_form(model.index)[0] <= words
        a, b = model.query(Q), loaded.query(Q)
        np.testing.assert_array_equal(a.get_indices(), b.get_indices())
        np.testing.assert_array_equal(a.get_offsets(), b.get_offsets())
        assert a.get_counts()[:150].min() >= 1
    S = sparse(2000, 300, 0.04)
    lsh = MinHashLSH(n_hash_tables=8, n_hashes=4, seed=9)
    model = lsh.fit(S)
    path = os.path.join(tmp_path, "mh.npz")
    model.save(path)
    loaded = MinHashLSHModel.load(path)
    assert _key_form(model.index) == (2, 3) == _key_form(loaded.index)                # 4 x 9 bits
    a, b = model.query(S[:200]), loaded.query(S[:200])
    np.testing.assert_array_equal(a.get_indices(), b.get_indices())
    np.testing.assert_array_equal(a.get_offsets(), b.get_offsets())
    # column ids beyond n_features: the fit falls back to plain keys, and so does the load
    wide, wide_q = S.copy(), S[:200].copy()
    wide.indices = (wide.indices + 5).astype(np.int32)                                 # ids up to 304 >= 300 = n_features
    wide_q.indices = (wide_q.indices + 5).astype(np.int32)
    model = lsh.fit(wide)
    path = os.path.join(tmp_path, "mh_wide.npz")
    model.save(path)
    loaded = MinHashLSHModel.load(path)
    assert _key_form(model.index) == (4, 0) == _key_form(loaded.index)
    a, b = model.query(wide_q), loaded.query(wide_q)
    np.testing.assert_array_equal(a.get_indices(), b.get_indices())
    np.testing.assert_array_equal(a.get_offsets(), b.get_offsets())


# ---------------------------------------------------------------- the reference's import name
def test_reference_import_name_runs_the_reference_usage(tmp_path):
    """A caller written against rishic3/cuLSH (README usage; python/tests/test_rplsh.py:145-174) runs
    unchanged through `import culsh`: fit, query, fit_query == fit + query, save / load."""
    from culsh import RPLSH, RPLSHModel
    from culsh._culsh_core import Candidates

    X = dense(1500, 48, np.float32, seed=3)
    Q = X[:60]
    lsh = RPLSH(n_hash_tables=8, n_hashes=6, seed=5)
    model = lsh.fit(X)
    assert isinstance(model, RPLSHModel)
    cand = model.query(Q)
    assert isinstance(cand, Candidates)
    both = RPLSH(n_hash_tables=8, n_hashes=6, seed=5).fit_query(X)
    again = model.query(X)
    np.testing.assert_array_equal(both.get_indices(), again.get_indices())
    np.testing.assert_array_equal(both.get_offsets(), again.get_offsets())
    path = os.path.join(tmp_path, "model.npz")
    model.save(path)
    loaded = RPLSHModel.load(path)
    np.testing.assert_array_equal(loaded.query(Q).get_indices(), cand.get_indices())
    # every query finds itself
    off = cand.get_offsets().astype(np.int64)
    idx = cand.get_indices()
    assert all(q in idx[off[q]:off[q + 1]] for q in range(len(Q)))
