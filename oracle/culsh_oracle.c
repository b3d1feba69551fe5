/*
 * CPU restatement (plain C + OpenMP) of cuLSH's fit/query hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke()
 * and the cpu_baseline leg of bench.py may load it; the shipped library never does.
 *
 * It follows the reference's algorithm step by step (paths relative to the reference
 * checkout) so that it can serve both as a second, independent checker next to the
 * numpy restatement in culsh_oracle.py and as the timed CPU baseline ("port"):
 *
 *   hashing      rplsh/hash.cuh:23-48,92-129  pslsh/hash.cuh:25-47,104-142
 *                minhash/hash.cuh:69-128
 *   index build  core/fit.cuh:222-374   (LSD byte passes S-1..0 from the identity
 *                permutation, table grouping, boundary flags, scan, scatter)
 *   query        core/query.cuh:31-101 (binary search), :114-237 (count, prefix, gather),
 *                :245-279,:393-465 (per-query ascending sort, unique, compaction)
 *   fit_query    core/fit_query.cuh:30-55
 *
 * The GEMM (cuBLAS in the reference) is a float dot product here; its summation order
 * differs from any GPU's, which is why hash bits within 1e-5 relative of the decision
 * boundary are excluded from bit parity (see culsh_oracle.py).  Parity of the raw
 * random parameter stream (cuRAND XORWOW in the reference) is unpinned; parameters are
 * always passed in.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define MINHASH_PRIME 4294967291ull /* minhash/hash.cuh:17 */

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_free(void* p) { free(p); }

/* ---------------------------------------------------------------- hashing ---------- */

/* X_hash = X * P^T in float (rplsh/hash.cuh:110-113), then sig[t][row][h] = 1 iff the sign
 * bit of the float is clear (rplsh/hash.cuh:47). */
void oracle_rplsh_hash_f32(const float* X, const float* P, int n, int d, int T, int H,
                           uint8_t* sig) {
    const int TH = T * H;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < n; ++r) {
        const float* x = X + (size_t)r * d;
        for (int c = 0; c < TH; ++c) {
            const float* p = P + (size_t)c * d;
            float acc = 0.0f;
            for (int k = 0; k < d; ++k) acc += x[k] * p[k];
            uint32_t bits;
            memcpy(&bits, &acc, 4);
            int t = c / H, h = c % H;
            sig[(size_t)t * n * H + (size_t)r * H + h] = (uint8_t)((bits >> 31) ^ 1u);
        }
    }
}

/* The same function blocked for the registers and the vector units: P is repacked once into panels
 * of CB columns ([panel][feature][CB]), and a block of RB rows x CB columns is accumulated in
 * registers over all features.  Every output is still the sum of its products in feature order, one
 * rounding per product and per addition (no contraction in ISO C mode), so the result equals
 * oracle_rplsh_hash_f32 bit for bit; tests require that. */
void oracle_rplsh_hash_f32_blocked(const float* X, const float* P, int n, int d, int T, int H,
                                   uint8_t* sig) {
    enum { RB = 4, CB = 16 };
    const int TH = T * H;
    const int panels = (TH + CB - 1) / CB;
    float* Pp = (float*)calloc((size_t)panels * d * CB, sizeof(float));
    if (!Pp) {  /* no scratch: the plain way */
        oracle_rplsh_hash_f32(X, P, n, d, T, H, sig);
        return;
    }
    for (int c = 0; c < TH; ++c)
        for (int k = 0; k < d; ++k) Pp[((size_t)(c / CB) * d + k) * CB + c % CB] = P[(size_t)c * d + k];
#pragma omp parallel for schedule(static)
    for (int r0 = 0; r0 < n; r0 += RB) {
        const int rows = n - r0 < RB ? n - r0 : RB;
        const float* x[RB];
        for (int rr = 0; rr < RB; ++rr) x[rr] = X + (size_t)(r0 + (rr < rows ? rr : 0)) * d;  /* spare rows repeat the first */
        for (int p = 0; p < panels; ++p) {
            const float* pp = Pp + (size_t)p * d * CB;
            float acc[RB][CB];
            for (int rr = 0; rr < RB; ++rr)
                for (int j = 0; j < CB; ++j) acc[rr][j] = 0.0f;
            for (int k = 0; k < d; ++k)
                for (int rr = 0; rr < RB; ++rr) {
                    const float xv = x[rr][k];
                    for (int j = 0; j < CB; ++j) acc[rr][j] += xv * pp[(size_t)k * CB + j];
                }
            for (int rr = 0; rr < rows; ++rr)
                for (int j = 0; j < CB && p * CB + j < TH; ++j) {
                    const int c = p * CB + j;
                    uint32_t bits;
                    memcpy(&bits, &acc[rr][j], 4);
                    const int t = c / H, h = c % H;
                    sig[(size_t)t * n * H + (size_t)(r0 + rr) * H + h] = (uint8_t)((bits >> 31) ^ 1u);
                }
        }
    }
    free(Pp);
}

void oracle_rplsh_hash_f64(const double* X, const double* P, int n, int d, int T, int H,
                           uint8_t* sig) {
    const int TH = T * H;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < n; ++r) {
        const double* x = X + (size_t)r * d;
        for (int c = 0; c < TH; ++c) {
            const double* p = P + (size_t)c * d;
            double acc = 0.0;
            for (int k = 0; k < d; ++k) acc += x[k] * p[k];
            float f = (float)acc; /* narrowing keeps the sign (rplsh/hash.cuh:47) */
            uint32_t bits;
            memcpy(&bits, &f, 4);
            int t = c / H, h = c % H;
            sig[(size_t)t * n * H + (size_t)r * H + h] = (uint8_t)((bits >> 31) ^ 1u);
        }
    }
}

/* sig[t][row][h] = (int32)floor(X*P^T + b[t*H+h]) (pslsh/hash.cuh:46). */
void oracle_pslsh_hash_f32(const float* X, const float* P, const float* b, int n, int d, int T,
                           int H, int32_t* sig) {
    const int TH = T * H;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < n; ++r) {
        const float* x = X + (size_t)r * d;
        for (int c = 0; c < TH; ++c) {
            const float* p = P + (size_t)c * d;
            float acc = 0.0f;
            for (int k = 0; k < d; ++k) acc += x[k] * p[k];
            int t = c / H, h = c % H;
            sig[(size_t)t * n * H + (size_t)r * H + h] = (int32_t)floorf(acc + b[c]);
        }
    }
}

void oracle_pslsh_hash_f64(const double* X, const double* P, const double* b, int n, int d, int T,
                           int H, int32_t* sig) {
    const int TH = T * H;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < n; ++r) {
        const double* x = X + (size_t)r * d;
        for (int c = 0; c < TH; ++c) {
            const double* p = P + (size_t)c * d;
            double acc = 0.0;
            for (int k = 0; k < d; ++k) acc += x[k] * p[k];
            int t = c / H, h = c % H;
            sig[(size_t)t * n * H + (size_t)r * H + h] = (int32_t)floor(acc + b[c]);
        }
    }
}

/* sig[t][row][h] = min_j ((uint64)A*idx_j + B) mod p, empty row -> 0xFFFFFFFF
 * (minhash/hash.cuh:86-127). */
void oracle_minhash_mod(const int32_t* indices, const int32_t* indptr, const uint32_t* A,
                        const uint32_t* B, int n, int T, int H, uint64_t prime, uint32_t* sig) {
    const int TH = T * H;
#pragma omp parallel for schedule(dynamic, 256)
    for (int r = 0; r < n; ++r) {
        int s = indptr[r], e = indptr[r + 1];
        for (int c = 0; c < TH; ++c) {
            uint32_t m = 0xFFFFFFFFu;
            for (int j = s; j < e; ++j) {
                uint64_t v = (uint64_t)A[c] * (uint32_t)indices[j] + (uint64_t)B[c];
                uint32_t hv = (uint32_t)(v % prime);
                if (hv < m) m = hv;
            }
            int t = c / H, h = c % H;
            sig[(size_t)t * n * H + (size_t)r * H + h] = m;
        }
    }
}

/* the reference's prime */
void oracle_minhash(const int32_t* indices, const int32_t* indptr, const uint32_t* A,
                    const uint32_t* B, int n, int T, int H, uint32_t* sig) {
    oracle_minhash_mod(indices, indptr, A, B, n, T, H, MINHASH_PRIME, sig);
}

/* ---------------------------------------------------------------- index build ------ */

typedef struct {
    int32_t* all_candidate_indices;    /* [n_total_candidates] */
    uint8_t* all_bucket_signatures;    /* [n_total_buckets * sig_nbytes] */
    int32_t* bucket_candidate_offsets; /* [n_total_buckets + 1] */
    int32_t* table_bucket_offsets;     /* [n_hash_tables + 1] */
    int32_t* item_to_bucket;           /* [n * T] or NULL */
    int32_t n_total_candidates, n_total_buckets, n_hash_tables, n_hashes, sig_nbytes;
} oracle_index;

void oracle_index_free(oracle_index* ix) {
    free(ix->all_candidate_indices);
    free(ix->all_bucket_signatures);
    free(ix->bucket_candidate_offsets);
    free(ix->table_bucket_offsets);
    free(ix->item_to_bucket);
    memset(ix, 0, sizeof(*ix));
}

/* One stable 8-bit counting pass over the rows of one table (the role of the
 * extract_byte_key_kernel + SortPairs(0..8) pair at core/fit.cuh:265-272). */
static void lsd_pass(const uint8_t* sig_t, int S, int byte_idx, const uint32_t* in, uint32_t* out,
                     int n) {
    size_t count[257];
    memset(count, 0, sizeof(count));
    for (int i = 0; i < n; ++i) count[sig_t[(size_t)in[i] * S + byte_idx] + 1]++;
    for (int b = 0; b < 256; ++b) count[b + 1] += count[b];
    for (int i = 0; i < n; ++i) out[count[sig_t[(size_t)in[i] * S + byte_idx]]++] = in[i];
}

/* core::detail::fit_index (core/fit.cuh:222-374).  The reference sorts all (table,row)
 * items at once and regroups them with a final stable pass on the table id
 * (fit.cuh:278-282); a stable sort inside each table block is the same permutation, and
 * lets the tables run on separate threads. */
int oracle_fit_index(const uint8_t* X_sig, int n, int T, int H, int S, int want_item_to_bucket,
                     oracle_index* out) {
    memset(out, 0, sizeof(*out));
    size_t N = (size_t)n * T;
    int32_t* cand = (int32_t*)malloc((N ? N : 1) * sizeof(int32_t));
    uint8_t* flags = (uint8_t*)malloc(N ? N : 1);
    int32_t* per_table_buckets = (int32_t*)calloc(T + 1, sizeof(int32_t));
    if (!cand || !flags || !per_table_buckets) return -1;

#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < T; ++t) {
        const uint8_t* sig_t = X_sig + (size_t)t * n * S;
        uint32_t* a = (uint32_t*)malloc((n ? n : 1) * sizeof(uint32_t));
        uint32_t* b = (uint32_t*)malloc((n ? n : 1) * sizeof(uint32_t));
        for (int i = 0; i < n; ++i) a[i] = (uint32_t)i; /* thrust::sequence, fit.cuh:254 */
        for (int byte_idx = S - 1; byte_idx >= 0; --byte_idx) {
            lsd_pass(sig_t, S, byte_idx, a, b, n);
            uint32_t* tmp = a;
            a = b;
            b = tmp;
        }
        int32_t nb = 0;
        for (int i = 0; i < n; ++i) {
            cand[(size_t)t * n + i] = (int32_t)a[i]; /* fit.cuh:177 */
            int head = (i == 0) || memcmp(sig_t + (size_t)a[i] * S, sig_t + (size_t)a[i - 1] * S,
                                          S) != 0; /* fit.cuh:110-143 */
            flags[(size_t)t * n + i] = (uint8_t)head;
            nb += head;
        }
        per_table_buckets[t + 1] = nb;
        free(a);
        free(b);
    }
    /* exclusive scan of bucket flags + selection at table starts (fit.cuh:305-326) */
    for (int t = 0; t < T; ++t) per_table_buckets[t + 1] += per_table_buckets[t];
    int32_t B = per_table_buckets[T];

    out->all_candidate_indices = cand;
    out->table_bucket_offsets = per_table_buckets; /* [T] holds the terminator, fit.cuh:353 */
    out->bucket_candidate_offsets = (int32_t*)malloc(((size_t)B + 1) * sizeof(int32_t));
    out->all_bucket_signatures = (uint8_t*)malloc((size_t)B * S + 1);
    if (want_item_to_bucket) out->item_to_bucket = (int32_t*)malloc((N ? N : 1) * sizeof(int32_t));
    out->bucket_candidate_offsets[B] = (int32_t)N; /* fit.cuh:355 */

#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < T; ++t) {
        const uint8_t* sig_t = X_sig + (size_t)t * n * S;
        int32_t bkt = per_table_buckets[t] - 1;
        for (int i = 0; i < n; ++i) {
            size_t pos = (size_t)t * n + i;
            int32_t row = cand[pos];
            if (flags[pos]) { /* fit.cuh:187-206 */
                ++bkt;
                out->bucket_candidate_offsets[bkt] = (int32_t)pos;
                memcpy(out->all_bucket_signatures + (size_t)bkt * S, sig_t + (size_t)row * S, S);
            }
            if (want_item_to_bucket) out->item_to_bucket[(size_t)row * T + t] = bkt; /* :180-185 */
        }
    }
    free(flags);
    out->n_total_candidates = (int32_t)N;
    out->n_total_buckets = B;
    out->n_hash_tables = T;
    out->n_hashes = H;
    out->sig_nbytes = S;
    return 0;
}

/* ---------------------------------------------------------------- query ------------ */

typedef struct {
    int32_t* query_candidate_indices;  /* [n_total_candidates] */
    uint64_t* query_candidate_counts;  /* [n_queries] */
    uint64_t* query_candidate_offsets; /* [n_queries + 1] */
    int32_t n_queries;
    uint64_t n_total_candidates;
    uint64_t n_raw_candidates; /* duplicates included (size of the gather) */
} oracle_candidates;

void oracle_candidates_free(oracle_candidates* c) {
    free(c->query_candidate_indices);
    free(c->query_candidate_counts);
    free(c->query_candidate_offsets);
    memset(c, 0, sizeof(*c));
}

/* find_bucket_in_table (core/query.cuh:31-60) */
static int find_bucket(const uint8_t* bsig, int lo, int hi_excl, const uint8_t* q, int S) {
    int hi = hi_excl - 1;
    while (lo <= hi) {
        int mid = lo + (hi - lo) / 2;
        int cmp = memcmp(q, bsig + (size_t)mid * S, S); /* unsigned byte-wise, byte 0 first */
        if (cmp == 0) return mid;
        if (cmp < 0)
            hi = mid - 1;
        else
            lo = mid + 1;
    }
    return -1;
}

/* find_matching_buckets_kernel (core/query.cuh:72-101): matched[q*T + t] */
void oracle_find_matching_buckets(const uint8_t* Q_sig, int nq, int S, const oracle_index* ix,
                                  int32_t* matched) {
    int T = ix->n_hash_tables;
#pragma omp parallel for schedule(static)
    for (int q = 0; q < nq; ++q)
        for (int t = 0; t < T; ++t)
            matched[(size_t)q * T + t] =
                find_bucket(ix->all_bucket_signatures, ix->table_bucket_offsets[t],
                            ix->table_bucket_offsets[t + 1],
                            Q_sig + (size_t)t * nq * S + (size_t)q * S, S);
}

static int cmp_i32(const void* a, const void* b) {
    int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
    return (x > y) - (x < y);
}

/* query_from_matched_buckets (core/query.cuh:290-478) */
int oracle_query_from_matched_buckets(const int32_t* matched, int nq, const oracle_index* ix,
                                      oracle_candidates* out) {
    memset(out, 0, sizeof(*out));
    int T = ix->n_hash_tables;
    const int32_t* bco = ix->bucket_candidate_offsets;
    uint64_t* raw_off = (uint64_t*)malloc(((size_t)nq + 1) * sizeof(uint64_t));
    out->query_candidate_counts = (uint64_t*)calloc(nq ? nq : 1, sizeof(uint64_t));
    out->query_candidate_offsets = (uint64_t*)calloc((size_t)nq + 1, sizeof(uint64_t));
    out->n_queries = nq;
    raw_off[0] = 0;
    for (int q = 0; q < nq; ++q) { /* count + aggregate + scan, query.cuh:114-183,:330-336 */
        uint64_t c = 0;
        for (int t = 0; t < T; ++t) {
            int32_t b = matched[(size_t)q * T + t];
            if (b != -1) c += (uint64_t)(bco[b + 1] - bco[b]);
        }
        raw_off[q + 1] = raw_off[q] + c;
    }
    uint64_t R = raw_off[nq];
    out->n_raw_candidates = R;
    if (R == 0) { /* query.cuh:358-365 */
        free(raw_off);
        return 0;
    }
    int32_t* raw = (int32_t*)malloc(R * sizeof(int32_t));
    if (!raw) return -1;
#pragma omp parallel for schedule(dynamic, 16)
    for (int q = 0; q < nq; ++q) {
        int32_t* seg = raw + raw_off[q];
        size_t m = 0;
        for (int t = 0; t < T; ++t) { /* collect_candidates_kernel, query.cuh:199-237 */
            int32_t b = matched[(size_t)q * T + t];
            if (b == -1) continue;
            int32_t len = bco[b + 1] - bco[b];
            memcpy(seg + m, ix->all_candidate_indices + bco[b], (size_t)len * sizeof(int32_t));
            m += len;
        }
        qsort(seg, m, sizeof(int32_t), cmp_i32); /* segmented sort, query.cuh:393-402 */
        size_t u = 0;
        for (size_t i = 0; i < m; ++i) /* mark_unique + fix_boundaries, query.cuh:245-279 */
            if (i == 0 || seg[i] != seg[i - 1]) seg[u++] = seg[i];
        out->query_candidate_counts[q] = u; /* segmented reduce, query.cuh:415-422 */
    }
    for (int q = 0; q < nq; ++q) /* query.cuh:425-431 */
        out->query_candidate_offsets[q + 1] =
            out->query_candidate_offsets[q] + out->query_candidate_counts[q];
    uint64_t U = out->query_candidate_offsets[nq];
    out->n_total_candidates = U;
    out->query_candidate_indices = (int32_t*)malloc((U ? U : 1) * sizeof(int32_t));
#pragma omp parallel for schedule(static)
    for (int q = 0; q < nq; ++q) /* compaction, query.cuh:458-465 */
        memcpy(out->query_candidate_indices + out->query_candidate_offsets[q], raw + raw_off[q],
               out->query_candidate_counts[q] * sizeof(int32_t));
    free(raw);
    free(raw_off);
    return 0;
}

/* query_index (core/query.cuh:490-522) */
int oracle_query_index(const uint8_t* Q_sig, int nq, int S, const oracle_index* ix,
                       oracle_candidates* out) {
    int32_t* matched = (int32_t*)malloc(((size_t)nq * ix->n_hash_tables + 1) * sizeof(int32_t));
    if (!matched) return -1;
    oracle_find_matching_buckets(Q_sig, nq, S, ix, matched);
    int rc = oracle_query_from_matched_buckets(matched, nq, ix, out);
    free(matched);
    return rc;
}

/* fit_query (core/fit_query.cuh:30-55) */
int oracle_fit_query(const uint8_t* X_sig, int n, int T, int H, int S, oracle_candidates* out) {
    oracle_index ix;
    int rc = oracle_fit_index(X_sig, n, T, H, S, 1, &ix);
    if (rc) return rc;
    rc = oracle_query_from_matched_buckets(ix.item_to_bucket, n, &ix, out);
    oracle_index_free(&ix);
    return rc;
}
