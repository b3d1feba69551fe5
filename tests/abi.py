"""
Test-side helpers: the C-ABI driver of the package plus bit-exact comparisons against the oracle's
dataclasses.
"""

from __future__ import annotations

import numpy as np

from culsh_amd.abi import Ctx, dev, hp, ptr, torch  # noqa: F401  (re-exported for the tests)


def assert_index_matches(got: dict, exp) -> None:
    """got: Ctx.index_arrays dict; exp: oracle Index dataclass. Bit-exact."""
    assert got["n_total_buckets"] == exp.n_total_buckets
    assert got["n_total_candidates"] == exp.n_total_candidates
    assert got["sig_nbytes"] == exp.sig_nbytes
    assert got["n_hash_tables"] == exp.n_hash_tables
    np.testing.assert_array_equal(got["table_bucket_offsets"], exp.table_bucket_offsets)
    np.testing.assert_array_equal(got["bucket_candidate_offsets"], exp.bucket_candidate_offsets)
    np.testing.assert_array_equal(got["all_bucket_signatures"], exp.all_bucket_signatures)
    np.testing.assert_array_equal(got["all_candidate_indices"], exp.all_candidate_indices)


def assert_candidates_match(got: dict, exp) -> None:
    """got: Ctx.candidates_arrays dict; exp: oracle Candidates dataclass. Bit-exact."""
    assert got["n_queries"] == exp.n_queries
    assert got["n_total_candidates"] == exp.n_total_candidates
    np.testing.assert_array_equal(got["counts"], exp.query_candidate_counts)
    np.testing.assert_array_equal(got["offsets"], exp.query_candidate_offsets)
    np.testing.assert_array_equal(got["indices"], exp.query_candidate_indices)
