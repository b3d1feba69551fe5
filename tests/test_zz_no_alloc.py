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


@pytest.mark.parametrize("kind", ["rplsh", "pslsh"])
def test_static_lookup_allocates_nothing(ctx, kind):
    """Around the static call nothing moves that an allocation would move: the library's count of calls
    into the HIP allocator (hipMalloc, hipHostMalloc, hipFree, hipEventCreate), the context's scratch
    arena (size, bytes in use, blocks beside it) and the device's free memory.  Also with per-kernel
    timing switched on (the allocating lookup then takes events from a pool or creates them), and for
    two calls issued back to back without a wait in between, followed by one culsh_ctx_synchronize."""
    import ctypes as C

    import torch

    from abi import dev, ptr
    from culsh_amd import _lib as L

    print("[case] static lookup allocates nothing", kind, flush=True)
    rng = np.random.default_rng(99)
    T, n, H = 5, 3000, 3
    sig = _sigs(rng, T, n, H, kind)
    ih, _ = ctx.core_fit_index(sig, H)
    exp_ix = o.fit_index(sig, H)
    qa, qb = _sigs(rng, T, 400, H, kind), _sigs(rng, T, 150, H, kind)
    qa[:, :200] = sig[:, rng.integers(0, n, 200)]
    qb[:, :75] = sig[:, rng.integers(0, n, 75)]
    S = qa.dtype.itemsize * H
    da, db = dev(qa.view(np.uint8).reshape(-1)), dev(qb.view(np.uint8).reshape(-1))
    ma = torch.empty(400 * T, dtype=torch.int32, device="cuda")
    mb = torch.empty(150 * T, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()

    def state():
        arena = (C.c_uint64 * 4)()
        L.check(ctx.lib.culsh_debug_arena_state(ctx.h, arena))
        return int(ctx.lib.culsh_debug_allocation_calls()), tuple(arena), torch.cuda.mem_get_info()[0]

    for timing in (0, 1):
        L.check(ctx.lib.culsh_profile_enable(ctx.h, timing))
        before = state()
        L.check(ctx.lib.culsh_core_find_matching_buckets_static(ctx.h, ptr(da), 400, S, ih, ptr(ma)))
        L.check(ctx.lib.culsh_core_find_matching_buckets_static(ctx.h, ptr(db), 150, S, ih, ptr(mb)))   # no wait in between
        ctx.synchronize()
        assert state() == before
        np.testing.assert_array_equal(ma.cpu().numpy(), o.find_matching_buckets(qa, exp_ix))
        np.testing.assert_array_equal(mb.cpu().numpy(), o.find_matching_buckets(qb, exp_ix))
    L.check(ctx.lib.culsh_profile_enable(ctx.h, 0))
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
    T, n, H = 2, 100, 40                        # 40 opaque bytes -> 10 key words per signature
    sig = rng.integers(0, 2, size=(T, n, H), dtype=np.uint8)
    ih, _ = ctx.core_fit_index(sig, H)
    nq = (1 << 20) // (T * 10) + 1              # opaque byte keys: 10 words each
    q = torch.zeros(T * nq * H, dtype=torch.uint8, device="cuda")
    m = torch.empty(T * nq, dtype=torch.int32, device="cuda")
    rc = ctx.lib.culsh_core_find_matching_buckets_static(ctx.h, q.data_ptr(), nq, H, ih, m.data_ptr())
    assert rc == L.ERR_LIMIT and "static" in L.last_error()
    ctx.free_index(ih)
