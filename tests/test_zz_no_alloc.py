"""
The entry point that allocates nothing: culsh_core_find_matching_buckets_static against
culsh_core_find_matching_buckets (and the oracle) on the same inputs, through the C ABI.  Two calls
in a row, the second with fewer queries (the workspace keeps the first call's key words), for every
key encoding; sizes beyond the workspace are refused.
"""

import numpy as np
import pytest

from oracle import culsh_oracle as o

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from abi import Ctx

    c = Ctx(0)
    yield c
    c.close()


def _sigs(rng, T, n, H, kind):
    if kind == "rplsh":
        return rng.integers(0, 2, size=(T, n, H), dtype=np.uint8)
    if kind == "pslsh":
        return rng.integers(-3, 4, size=(T, n, H)).astype(np.int32)
    v = rng.integers(0, 6, size=(T, n, H)).astype(np.uint32)
    return (v * np.uint32(0x01000193)) ^ np.uint32(0x80000001)


@pytest.mark.parametrize("kind", ["rplsh", "pslsh", "minhash"])
def test_static_lookup_matches_allocating_lookup(ctx, kind):
    print("[case] static lookup", kind, flush=True)
    rng = np.random.default_rng(2024)
    T, n, H = 6, 4000, 3
    sig = _sigs(rng, T, n, H, kind)
    ih, _ = ctx.core_fit_index(sig, H)
    exp_ix = o.fit_index(sig, H)
    for nq in (700, 90):                       # the second call is smaller than the first
        qsig = _sigs(rng, T, nq, H, kind)
        qsig[:, : nq // 2] = sig[:, rng.integers(0, n, nq // 2)]   # half of the queries are fitted rows
        want = ctx.core_find_matching_buckets(qsig, ih)
        got = ctx.core_find_matching_buckets(qsig, ih, static=True)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(got, o.find_matching_buckets(qsig, exp_ix))
        assert (got >= 0).sum() >= T * (nq // 2)
    ctx.free_index(ih)


def test_static_lookup_after_family_fit(ctx):
    """An index whose keys are compressed ranks (p-stable fit): the static lookup converts query
    signatures with the index's tables, as the allocating one does."""
    print("[case] static lookup pslsh fit", flush=True)
    rng = np.random.default_rng(7)
    n, d, T, H = 3000, 16, 4, 4
    X = rng.standard_normal((n, d)).astype(np.float32)
    P = (rng.standard_normal((T * H, d)) / 4).astype(np.float32)
    b = rng.uniform(0.01, 1.0, T * H).astype(np.float32)
    ih = ctx.pslsh_fit(X, T, H, 4, seed=3, P=P, b=b)
    for nq in (500, 33):
        Q = X[rng.integers(0, n, nq)] + rng.normal(0, 0.05, (nq, d)).astype(np.float32)
        qsig = ctx.pslsh_hash(Q.astype(np.float32), P, b, T, H)
        want = ctx.core_find_matching_buckets(qsig, ih)
        got = ctx.core_find_matching_buckets(qsig, ih, static=True)
        np.testing.assert_array_equal(got, want)
        assert (got >= 0).any()
    ctx.free_index(ih)


def test_static_lookup_refuses_sizes_beyond_the_workspace(ctx):
    import ctypes as C

    import torch

    from culsh_amd import _lib as L

    rng = np.random.default_rng(1)
    T, n, H = 2, 100, 40                        # 40 sign bytes -> 2 key words per signature
    sig = rng.integers(0, 2, size=(T, n, H), dtype=np.uint8)
    ih, _ = ctx.core_fit_index(sig, H)
    nq = (1 << 20) // (T * 10) + 1              # opaque byte keys: 10 words each
    q = torch.zeros(T * nq * H, dtype=torch.uint8, device="cuda")
    m = torch.empty(T * nq, dtype=torch.int32, device="cuda")
    rc = ctx.lib.culsh_core_find_matching_buckets_static(ctx.h, q.data_ptr(), nq, H, ih, m.data_ptr())
    assert rc == L.ERR_LIMIT and "static" in L.last_error()
    ctx.free_index(ih)
