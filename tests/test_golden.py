"""
Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU part: the fixtures are what the oracle produces today (no silent drift), their
floating-point inputs really are summation-order independent, and their candidate lists
equal a brute-force union over tables of the rows whose stored signature equals the
query's (independent of the oracle's sort / lookup / dedup code).
GPU part: the HIP path reproduces every stored array bit for bit through the C ABI.
"""
import os

import numpy as np
import pytest

from oracle import culsh_oracle as o

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLDEN, name)) as z:   # allow_pickle stays False
        return {k: z[k] for k in z.files}


def brute_force_candidates(sig, qsig):
    T, n, _ = sig.shape
    nq = qsig.shape[1]
    lists = []
    for q in range(nq):
        hit = np.zeros(n, dtype=bool)
        for t in range(T):
            hit |= (sig[t] == qsig[t, q]).all(axis=1)
        lists.append(np.flatnonzero(hit).astype(np.int32))
    counts = np.array([len(x) for x in lists], dtype=np.uint64)
    offsets = np.zeros(nq + 1, dtype=np.uint64)
    offsets[1:] = np.cumsum(counts)
    return (np.concatenate(lists) if offsets[-1] else np.zeros(0, np.int32)), counts, offsets


def check_index(g, ix):
    for k in ("all_candidate_indices", "all_bucket_signatures", "bucket_candidate_offsets", "table_bucket_offsets"):
        np.testing.assert_array_equal(np.asarray(getattr(ix, k)).reshape(-1), g["ix_" + k].reshape(-1), err_msg=k)


def check_cands(g, prefix, c):
    np.testing.assert_array_equal(c.query_candidate_indices, g[prefix + "indices"])
    np.testing.assert_array_equal(c.query_candidate_counts, g[prefix + "counts"])
    np.testing.assert_array_equal(c.query_candidate_offsets, g[prefix + "offsets"])


# ------------------------------------------------------------------------------- CPU
def test_rplsh_fixture_matches_oracle_and_brute_force(c_oracle):
    g = load("rplsh_small.npz")
    T, H = int(g["T"]), int(g["H"])
    # exactness of the inputs: fp32 and fp64 products agree, so any summation order does
    p32 = g["X"] @ g["P"].T
    np.testing.assert_array_equal(p32.astype(np.float64), g["X"].astype(np.float64) @ g["P"].astype(np.float64).T)
    assert (p32 == 0).any()   # the zero rule is exercised
    np.testing.assert_array_equal(o.rplsh_hash(g["X"], g["P"], T, H), g["sig"])
    np.testing.assert_array_equal(o.rplsh_hash(g["Q"], g["P"], T, H), g["qsig"])
    np.testing.assert_array_equal(c_oracle.rplsh_hash(g["X"], g["P"], T, H), g["sig"])
    # sign rule restated: bit = 1 unless the projection is negative (or -0)
    np.testing.assert_array_equal(g["sig"].transpose(1, 0, 2).reshape(len(g["X"]), T * H),
                                  (~np.signbit(p32)).astype(np.uint8))
    ix = o.fit_index(g["sig"], H)
    check_index(g, ix)
    check_cands(g, "q_", o.query_index(g["qsig"], ix))
    check_cands(g, "fq_", o.fit_query(g["sig"], H))
    bi, bc, bo = brute_force_candidates(g["sig"], g["qsig"])
    np.testing.assert_array_equal(bi, g["q_indices"])
    np.testing.assert_array_equal(bc, g["q_counts"])
    np.testing.assert_array_equal(bo, g["q_offsets"])
    bi, bc, bo = brute_force_candidates(g["sig"], g["sig"])
    np.testing.assert_array_equal(bi, g["fq_indices"])


def test_pslsh_fixture_matches_oracle_and_brute_force(c_oracle):
    g = load("pslsh_small.npz")
    T, H = int(g["T"]), int(g["H"])
    v32 = g["X"] @ g["P"].T + g["b"][None, :]
    v64 = g["X"].astype(np.float64) @ g["P"].astype(np.float64).T + g["b"].astype(np.float64)[None, :]
    np.testing.assert_array_equal(v32.astype(np.float64), v64)
    np.testing.assert_array_equal(o.pslsh_hash(g["X"], g["P"], g["b"], T, H), g["sig"])
    np.testing.assert_array_equal(o.pslsh_hash(g["Q"], g["P"], g["b"], T, H), g["qsig"])
    np.testing.assert_array_equal(c_oracle.pslsh_hash(g["X"], g["P"], g["b"], T, H), g["sig"])
    np.testing.assert_array_equal(g["sig"].transpose(1, 0, 2).reshape(len(g["X"]), T * H),
                                  np.floor(v64).astype(np.int32))
    ix = o.fit_index(g["sig"], H)
    check_index(g, ix)
    check_cands(g, "q_", o.query_index(g["qsig"], ix))
    check_cands(g, "fq_", o.fit_query(g["sig"], H))
    bi, bc, bo = brute_force_candidates(g["sig"], g["qsig"])
    np.testing.assert_array_equal(bi, g["q_indices"])
    np.testing.assert_array_equal(bo, g["q_offsets"])
    bi, bc, bo = brute_force_candidates(g["sig"], g["sig"])
    np.testing.assert_array_equal(bi, g["fq_indices"])
    np.testing.assert_array_equal(bo, g["fq_offsets"])


def test_minhash_fixture_matches_oracle_and_brute_force(c_oracle):
    g = load("minhash_small.npz")
    T, H = int(g["T"]), int(g["H"])
    np.testing.assert_array_equal(o.minhash_hash(g["x_indices"], g["x_indptr"], g["A"], g["B"], T, H), g["sig"])
    np.testing.assert_array_equal(c_oracle.minhash_hash(g["x_indices"], g["x_indptr"], g["A"], g["B"], T, H), g["sig"])
    np.testing.assert_array_equal(o.minhash_hash(g["qcsr_indices"], g["qcsr_indptr"], g["A"], g["B"], T, H), g["qsig"])
    # big-int restatement of one row per kind (non-empty, empty)
    p = 4294967291
    for row in (0, 3, 17):
        idx = g["x_indices"][g["x_indptr"][row]:g["x_indptr"][row + 1]]
        for t in range(T):
            for h in range(H):
                a, b = int(g["A"][t * H + h]), int(g["B"][t * H + h])
                exp = min(((a * int(i) + b) % p for i in idx), default=0xFFFFFFFF)
                assert int(g["sig"][t, row, h]) == exp
    ix = o.fit_index(g["sig"], H)
    check_index(g, ix)
    check_cands(g, "q_", o.query_index(g["qsig"], ix))
    check_cands(g, "fq_", o.fit_query(g["sig"], H))
    bi, bc, bo = brute_force_candidates(g["sig"], g["qsig"])
    np.testing.assert_array_equal(bi, g["q_indices"])
    np.testing.assert_array_equal(bo, g["q_offsets"])
    bi, bc, bo = brute_force_candidates(g["sig"], g["sig"])
    np.testing.assert_array_equal(bi, g["fq_indices"])
    np.testing.assert_array_equal(bo, g["fq_offsets"])


# ------------------------------------------------------------------------------- GPU
@pytest.fixture(scope="module")
def ctx():
    from abi import Ctx

    c = Ctx(0)
    yield c
    c.close()


def gpu_index_equals(ctx, ih, g):
    got = ctx.index_arrays(ih)
    for k in ("all_candidate_indices", "all_bucket_signatures", "bucket_candidate_offsets", "table_bucket_offsets"):
        np.testing.assert_array_equal(np.asarray(got[k]).reshape(-1).view(np.uint8),
                                      g["ix_" + k].reshape(-1).view(np.uint8), err_msg=k)


def gpu_cands_equal(got, g, prefix):
    np.testing.assert_array_equal(got["indices"], g[prefix + "indices"])
    np.testing.assert_array_equal(got["counts"], g[prefix + "counts"])
    np.testing.assert_array_equal(got["offsets"], g[prefix + "offsets"])


@pytest.mark.gpu
def test_gpu_rplsh_reproduces_fixture(ctx):
    g = load("rplsh_small.npz")
    T, H = int(g["T"]), int(g["H"])
    np.testing.assert_array_equal(ctx.rplsh_hash(g["X"], g["P"], T, H), g["sig"])
    ih = ctx.rplsh_fit(g["X"], T, H, P=g["P"])
    gpu_index_equals(ctx, ih, g)
    gpu_cands_equal(ctx.rplsh_query(g["Q"], ih), g, "q_")
    gpu_cands_equal(ctx.rplsh_query(g["Q"], ih, batch_size=7), g, "q_")
    ctx.free_index(ih)
    gpu_cands_equal(ctx.rplsh_fit_query(g["X"], T, H, P=g["P"]), g, "fq_")


@pytest.mark.gpu
def test_gpu_pslsh_reproduces_fixture(ctx):
    g = load("pslsh_small.npz")
    T, H, w = int(g["T"]), int(g["H"]), int(g["window"])
    np.testing.assert_array_equal(ctx.pslsh_hash(g["X"], g["P"], g["b"], T, H), g["sig"])
    ih = ctx.pslsh_fit(g["X"], T, H, w, P=g["P"], b=g["b"])
    gpu_index_equals(ctx, ih, g)
    gpu_cands_equal(ctx.pslsh_query(g["Q"], ih), g, "q_")
    gpu_cands_equal(ctx.pslsh_query(g["Q"], ih, batch_size=9), g, "q_")
    ctx.free_index(ih)
    gpu_cands_equal(ctx.pslsh_fit_query(g["X"], T, H, w, P=g["P"], b=g["b"]), g, "fq_")


@pytest.mark.gpu
def test_gpu_minhash_reproduces_fixture(ctx):
    g = load("minhash_small.npz")
    T, H, d = int(g["T"]), int(g["H"]), int(g["n_features"])
    np.testing.assert_array_equal(
        ctx.minhash_compute(g["x_indices"], g["x_indptr"], g["A"], g["B"], T, H).view(np.uint32), g["sig"])
    ih = ctx.minhash_fit(g["x_indices"], g["x_indptr"], d, T, H, A=g["A"], B=g["B"])
    gpu_index_equals(ctx, ih, g)
    gpu_cands_equal(ctx.minhash_query(g["qcsr_indices"], g["qcsr_indptr"], ih), g, "q_")
    ctx.free_index(ih)
    gpu_cands_equal(ctx.minhash_fit_query(g["x_indices"], g["x_indptr"], d, T, H, A=g["A"], B=g["B"]), g, "fq_")
