#!/usr/bin/env python3
"""
Writes the fixtures in this directory (small .npz files, numpy arrays only).

The reference holds no golden vectors for this path: its tests build their expectations on
the fly from python/tests/ref_lsh.py.  These fixtures are produced by the CPU oracle in
oracle/ (which tests/test_oracle.py pins against independent formulations) on inputs chosen
so that every floating-point dot product is exact in fp32 whatever the summation order
(small integers, window a power of two, biases multiples of 1/8).  That makes the
signatures, bucket tables and candidate lists below exact expectations for any correct
implementation, including the hash-of-exactly-zero rule of RPLSH.

    python tests/golden/make_golden.py        # rewrites the .npz files
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import culsh_oracle as o  # noqa: E402


def index_dict(prefix, ix):
    return {prefix + k: getattr(ix, k) for k in
            ("all_candidate_indices", "all_bucket_signatures", "bucket_candidate_offsets", "table_bucket_offsets")}


def cand_dict(prefix, c):
    return {prefix + "indices": c.query_candidate_indices, prefix + "counts": c.query_candidate_counts,
            prefix + "offsets": c.query_candidate_offsets}


def rplsh():
    rng = np.random.default_rng(101)
    n, d, nq, T, H = 300, 24, 40, 5, 6
    X = rng.integers(-8, 9, size=(n, d)).astype(np.float32)
    X[7] = 0.0                       # a zero row: every projection is exactly +0 -> bit 1
    Q = X[rng.integers(0, n, size=nq)].copy()
    Q[::3] += rng.integers(-1, 2, size=Q[::3].shape).astype(np.float32)
    P = rng.integers(-4, 5, size=(T * H, d)).astype(np.float32)
    sig, qsig = o.rplsh_hash(X, P, T, H), o.rplsh_hash(Q, P, T, H)
    ix = o.fit_index(sig, H)
    out = dict(X=X, Q=Q, P=P, T=T, H=H, sig=sig, qsig=qsig)
    out.update(index_dict("ix_", ix))
    out.update(cand_dict("q_", o.query_index(qsig, ix)))
    out.update(cand_dict("fq_", o.fit_query(sig, H)))
    np.savez_compressed(os.path.join(HERE, "rplsh_small.npz"), **out)


def pslsh():
    rng = np.random.default_rng(202)
    n, d, nq, T, H, w = 300, 20, 40, 4, 3, 4
    X = rng.integers(-6, 7, size=(n, d)).astype(np.float32)
    Q = X[rng.integers(0, n, size=nq)].copy()
    Q[::2] += rng.integers(-1, 2, size=Q[::2].shape).astype(np.float32)
    P = (rng.integers(-4, 5, size=(T * H, d)) / float(w)).astype(np.float32)   # already divided by the window
    b = (rng.integers(1, 9, size=T * H) / 8.0).astype(np.float32)               # in (0, 1]
    sig, qsig = o.pslsh_hash(X, P, b, T, H), o.pslsh_hash(Q, P, b, T, H)
    ix = o.fit_index(sig, H)
    out = dict(X=X, Q=Q, P=P, b=b, T=T, H=H, window=w, sig=sig, qsig=qsig)
    out.update(index_dict("ix_", ix))
    out.update(cand_dict("q_", o.query_index(qsig, ix)))
    out.update(cand_dict("fq_", o.fit_query(sig, H)))
    np.savez_compressed(os.path.join(HERE, "pslsh_small.npz"), **out)


def minhash():
    rng = np.random.default_rng(303)
    n, d, nq, T, H = 250, 40, 30, 4, 2
    rows = [np.sort(rng.choice(d, size=rng.integers(0, 7), replace=False)) for _ in range(n)]
    rows[3] = np.array([], dtype=np.int64)   # an empty row hashes to 0xFFFFFFFF
    qrows = [rows[i] for i in rng.integers(0, n, size=nq)]
    def csr(rs):
        indptr = np.zeros(len(rs) + 1, dtype=np.int32)
        indptr[1:] = np.cumsum([len(r) for r in rs])
        return np.concatenate(rs).astype(np.int32) if indptr[-1] else np.zeros(0, np.int32), indptr
    xi, xp = csr(rows)
    qi, qp = csr(qrows)
    A, B = o.generate_hash_integers(11, T * H)
    sig, qsig = o.minhash_hash(xi, xp, A, B, T, H), o.minhash_hash(qi, qp, A, B, T, H)
    ix = o.fit_index(sig, H)
    out = dict(x_indices=xi, x_indptr=xp, qcsr_indices=qi, qcsr_indptr=qp, n_features=d, A=A, B=B, T=T, H=H,
               sig=sig, qsig=qsig)
    out.update(index_dict("ix_", ix))
    out.update(cand_dict("q_", o.query_index(qsig, ix)))
    out.update(cand_dict("fq_", o.fit_query(sig, H)))
    np.savez_compressed(os.path.join(HERE, "minhash_small.npz"), **out)


if __name__ == "__main__":
    rplsh()
    pslsh()
    minhash()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
