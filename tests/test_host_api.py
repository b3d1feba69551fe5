"""
Host-side behaviour of the Python layer that needs no GPU: argument validation and error
types (the reference's checks at python/culsh/rp_lsh.py:62-65, utils.py:28-29,
minhash_lsh.py:304-307), seed handling and recall helper.
"""

import numpy as np
import pytest
import scipy.sparse

import culsh_amd
from culsh_amd import MinHashLSH, PStableLSH, RPLSH
from culsh_amd.minhash_lsh import ensure_int32_indices
from culsh_amd.utils import DeviceCSR, compute_recall, get_array_info, resolve_seed


def test_public_names():
    assert sorted(culsh_amd.__all__) == sorted(
        ["RPLSH", "RPLSHModel", "MinHashLSH", "MinHashLSHModel", "PStableLSH", "PStableLSHModel"])


@pytest.mark.parametrize("cls", [RPLSH, MinHashLSH, PStableLSH])
def test_constructor_validation(cls):
    with pytest.raises(ValueError, match="n_hash_tables must be positive"):
        cls(n_hash_tables=0, n_hashes=4)
    with pytest.raises(ValueError, match="n_hashes must be positive"):
        cls(n_hash_tables=4, n_hashes=-1)
    est = cls(n_hash_tables=3, n_hashes=5, seed=11)
    assert (est.n_hash_tables, est.n_hashes, est.seed) == (3, 5, 11)
    assert 0 <= cls(n_hash_tables=1, n_hashes=1).seed < 2**63


def test_pstable_window_validation():
    with pytest.raises(ValueError, match="window_size must be positive"):
        PStableLSH(2, 2, window_size=0)
    assert PStableLSH(2, 2).window_size == "auto"
    assert PStableLSH(2, 2, window_size=7).window_size == 7


def test_auto_window_size_estimate():
    """python/tests/test_pslsh.py:243-255: unit-norm rows scaled by 100 -> window 100."""
    rng = np.random.default_rng(0)
    X = rng.standard_normal((500, 32))
    X = 100.0 * X / np.linalg.norm(X, axis=1, keepdims=True)
    assert PStableLSH._estimate_window_size(X.astype(np.float32)) in (99, 100)
    assert PStableLSH._estimate_window_size(X) in (99, 100)
    assert PStableLSH._estimate_window_size(np.zeros((4, 3))) == 1
    big = np.ones((20000, 4))                      # sampling branch
    assert PStableLSH._estimate_window_size(big) == 2


def test_array_info_and_seed():
    assert get_array_info(np.zeros((3, 4), np.float32)) == (3, 4, np.dtype(np.float32))
    with pytest.raises(ValueError, match="Expected 2D array, got 1D"):
        get_array_info(np.zeros(3))
    m = scipy.sparse.random(5, 7, density=0.3, format="csr")
    assert get_array_info(m)[:2] == (5, 7)
    assert resolve_seed(5) == 5 and isinstance(resolve_seed(None), int)


def test_int32_indices_required():
    bad = DeviceCSR(np.zeros(3, np.int64), np.zeros(2, np.int32), (1, 4))
    with pytest.raises(ValueError, match="requires int32 indices"):
        ensure_int32_indices(bad)
    ok = DeviceCSR(np.zeros(3, np.int32), np.zeros(2, np.int64), (1, 4))
    ind, ptr = ensure_int32_indices(ok)
    assert ptr.dtype == np.int32 and ind.dtype == np.int32


def test_compute_recall():
    assert compute_recall(np.array([1, 2, 3]), np.array([2, 3, 4, 5])) == 0.5
    assert compute_recall(np.array([1]), np.array([])) == 0.0
